#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.  Default: simulated 8-rank bf16 ring allreduce, 128 MiB per rank.

One "step" is one complete collective over the N simulated ranks (2N HBM buffers).  Inputs are resident in
HBM before the timed region.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--lowering stepwise|fused|fused_keep_inputs|both]
                    [--no-cpu] [--cpu-threads T]

`value` is algorithmic GB/s of the whole collective - the two-input byte model, 3b per reduce and 2b per copy,
(5(N-1)S + 2S for an allreduce) divided by the wall time of a step - for the step-wise replay (one launch per
schedule step; bytes moved == algorithmic bytes).  The fused lowering, which leaves identical memory while
moving fewer bytes, is reported under "fused".  `roofline` prices the dominant kernel from HIP-event timings
taken on the stream the kernels run on.  `cpu_baseline` times the CPU oracle (a C restatement of the same
schedule) on the host cores of this machine, on the same inputs, and its result is used to verify the GPU
output bit for bit.  Workload `mesh_oneshot_fp16_n8_sweep` reports latency and GB/s per message size.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HcommLocalReduceOnThread refuses PROD like the reference's (cpu_primitives_c_adpt.cc:37); the via_primitives leg of the
# PROD workload (config 5a) needs the library's extended mode, read once when the library first sees a reduce
os.environ.setdefault("HCOMM_GFX_ALLOW_PROD", "1")



def measured_traffic(workload, lowering):
    """L2 <-> fabric bytes per launch of the dominant kernel, from profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE
    and WRITE_SIZE (KiB per dispatch), each scaled by what the same counter reads for a plain copy of known size.
    Written by `python -m hcomm_amd.profiling traffic ...` from the counter CSVs; None for what was not profiled."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            e = json.load(f)["entries"].get("%s|%s" % (workload, lowering))
    except (OSError, ValueError, KeyError):
        return None
    if not e:
        return None
    return (e["fetch_kib"] * e["fetch_scale"] + e["write_kib"] * e["write_scale"]) * 1024


# name: (algorithm, ranks, elements per rank, dtype, op, data distribution)
WORKLOADS = {
    "ring_ar_bf16_n8_128MiB": ("ring_ar", 8, 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    "ring_ar_fp32_n8_4MiB": ("ring_ar", 8, 1048576, "fp32", "sum", "uniform[-1,1)"),
    "rhd_ar_int32_n16_128MiB_sum": ("rhd_ar", 16, 33554432, "int32", "sum", "ints[-2^20,2^20]"),
    "rhd_ar_int32_n16_128MiB_max": ("rhd_ar", 16, 33554432, "int32", "max", "ints[-2^20,2^20]"),
    "rhd_ar_int32_n16_128MiB_min": ("rhd_ar", 16, 33554432, "int32", "min", "ints[-2^20,2^20]"),
    "ring_rs_fp32_prod_n7_100M": ("ring_rs_stage", 7, 100000003, "fp32", "prod", "uniform[0.99,1.01]"),
    "ring_rs_int8_sum_n7_100M": ("ring_rs_stage", 7, 100000003, "int8", "sum", "ints[-8,8]"),
    "mesh_oneshot_fp16_n8_4MiB": ("mesh_oneshot", 8, 2097152, "fp16", "sum", "uniform[-1,1)"),
    "mesh_oneshot_fp16_n8_4KiB": ("mesh_oneshot", 8, 2048, "fp16", "sum", "uniform[-1,1)"),
    "local_reduce_ar_bf16_n8_128MiB": ("local_reduce", 8, 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    "chunk_mesh_ar_bf16_n8_128MiB": ("chunk_mesh", 8, 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    "nhr_ar_bf16_n8_128MiB": ("nhr", 8, 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    "nb_ar_bf16_n8_128MiB": ("nb", 8, 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    "local_reduce_rs_bf16_n8_16MiB": ("local_reduce_rs", 8, 8388608, "bf16", "sum", "normal(0,1)*1e-3"),
    # whole-message recursive doubling, the small-message allreduce inside a server
    "doubling_ar_fp16_n8_64KiB": ("doubling", 8, 32768, "fp16", "sum", "uniform[-1,1)"),
    # the executors' op-base loop around the ring template: user buffers <-> 200 MiB CCL buffers (the default size)
    "opbase_ring_ar_bf16_n8_128MiB": ("opbase_ring_ar", 8, 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    "opbase_ring_ar_bf16_n8_512MiB": ("opbase_ring_ar", 8, 268435456, "bf16", "sum", "normal(0,1)*1e-3"),
    # the ring executor's three-step allreduce: 4 servers x 8 ranks, NHR / ring between the servers
    "hier_nhr_ar_bf16_4x8_128MiB": ("hier_nhr", (4, 8), 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    "meshhier_ring_ar_bf16_2x8_128MiB": ("meshhier_ring_ar", (2, 8), 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    "meshhier_ring_ar_bf16_1x8_128MiB": ("meshhier_ring_ar", (1, 8), 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    "hier_ring_ar_bf16_2x8_128MiB": ("hier_ring_ar", (2, 8), 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    # the double-ring executor in op-base mode with DMA reduce: user buffers read and written directly, 200 MiB CCL buffers
    "dbring_ring_ar_bf16_1x8_128MiB": ("dbring_ring_ar", (1, 8), 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    "dbring_ring_ar_bf16_1x8_512MiB": ("dbring_ring_ar", (1, 8), 268435456, "bf16", "sum", "normal(0,1)*1e-3"),
    "dbring_nhr_ar_bf16_2x8_128MiB": ("dbring_nhr", (2, 8), 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    # the order-preserving reduce-scatter executor: plant into the peers' CCL output buffers, fold in rank order
    "order_preserved_rs_bf16_n8_16MiB": ("order_preserved_rs", 8, 8388608, "bf16", "sum", "normal(0,1)*1e-3"),
    # blocks of 16,777,214 bytes: nothing but block 0 sits on a 16-byte boundary (the kernel for unaligned operands)
    "order_preserved_rs_bf16_n8_16MiB_odd": ("order_preserved_rs", 8, 8388607, "bf16", "sum", "normal(0,1)*1e-3"),
    # the same executor at 32 KiB per rank: its plant branch and the branch it takes there (ReduceScatterHDStage)
    "order_preserved_rs_bf16_n8_32KiB": ("order_preserved_rs", 8, 16384, "bf16", "sum", "normal(0,1)*1e-3"),
    "order_preserved_small_rs_bf16_n8_32KiB": ("order_preserved_small", 8, 16384, "bf16", "sum", "normal(0,1)*1e-3"),
    # the order-preserving allreduce executor: plant with a borrowed slot, fold in rank order, mesh all-gather
    "order_preserved_ar_bf16_n8_128MiB": ("order_preserved_ar", 8, 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    # the double-ring reduce-scatter executor on one server with DMA reduce
    "dbring_rs_bf16_n8_16MiB": ("doublering_rs", 8, 8388608, "bf16", "sum", "normal(0,1)*1e-3"),
    # the same executor over 2 servers x 8 devices, ring between the servers (blocks of 8 MiB)
    "dbringhier_ring_rs_bf16_2x8_8MiB": ("doublering_hier_rs", (2, 8), 4194304, "bf16", "sum", "normal(0,1)*1e-3"),
    # and over 2 super pods x 2 servers x 8 devices, ring at both levels (blocks of 4 MiB)
    "dbringhier_ring_rs_bf16_2x2x8_4MiB": ("doublering_hier_rs", (2, 2, 8), 2097152, "bf16", "sum", "normal(0,1)*1e-3"),
    # the order-preserving allreduce executor over two levels: plant + fold inside the servers, then between them
    "ophier_ring_ar_bf16_2x8_128MiB": ("ophier_ring_ar", (2, 8), 67108864, "bf16", "sum", "normal(0,1)*1e-3"),
    "ophierrs_ring_rs_bf16_2x8_8MiB": ("ophierrs_ring_rs_stage", (2, 8), 4194304, "bf16", "sum", "normal(0,1)*1e-3"),
    # the ring / mesh reduce-scatter executors over two levels in op-base mode (blocks of 16 MiB, 2 x 8 ranks)
    "hierrs_ring_rs_bf16_2x8_16MiB": ("hierrs_ring_rs_stage", (2, 8), 8388608, "bf16", "sum", "normal(0,1)*1e-3"),
    "meshhierrs_ring_rs_bf16_1x8_16MiB": ("meshhierrs_ring_rs_stage", (1, 8), 8388608, "bf16", "sum", "normal(0,1)*1e-3"),
    "nhr_oneshot_ar_bf16_n8_256KiB": ("nhr_oneshot", 8, 131072, "bf16", "sum", "normal(0,1)*1e-3"),
    "mesh_oneshot_fp16_n8_sweep": ("mesh_oneshot", 8, None, "fp16", "sum", "uniform[-1,1)"),
}


def make_inputs(torch, dev, n, count, dtname, seed=1234):
    """Seeded synthetic inputs on the GPU, returned as uint8 byte tensors (one per rank)."""
    gen = torch.Generator(device=dev)
    out = []
    for r in range(n):
        gen.manual_seed(seed + r)
        if dtname == "bf16":
            x = (torch.randn(count, generator=gen, device=dev, dtype=torch.float32) * 1e-3).to(torch.bfloat16)
        elif dtname == "fp16":
            x = (torch.rand(count, generator=gen, device=dev, dtype=torch.float32) * 2 - 1).to(torch.float16)
        elif dtname == "fp32":
            x = torch.rand(count, generator=gen, device=dev, dtype=torch.float32) * 2 - 1
        elif dtname == "fp32prod":
            x = torch.rand(count, generator=gen, device=dev, dtype=torch.float32) * 0.02 + 0.99
        elif dtname == "int32":
            x = torch.randint(-(1 << 20), (1 << 20) + 1, (count,), generator=gen, device=dev, dtype=torch.int32)
        elif dtname == "int8":
            x = torch.randint(-8, 9, (count,), generator=gen, device=dev, dtype=torch.int8)
        else:
            raise ValueError(dtname)
        out.append(x.view(torch.uint8).clone())
        del x
    return out


# what the default run appends to its line, beside the headline: (workload, steps) of the other BASELINE configs
CONFIG_LINE = [("ring_ar_fp32_n8_4MiB", 50), ("rhd_ar_int32_n16_128MiB_sum", 10), ("rhd_ar_int32_n16_128MiB_max", 10),
               ("rhd_ar_int32_n16_128MiB_min", 10), ("mesh_oneshot_fp16_n8_4KiB", 100), ("mesh_oneshot_fp16_n8_4MiB", 100),
               ("ring_rs_fp32_prod_n7_100M", 10), ("ring_rs_int8_sum_n7_100M", 10)]
MEMORY_SIDE_CACHE_BYTES = 256 << 20


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--lowering", default="both", choices=["stepwise", "fused", "fused_keep_inputs", "both"])
    ap.add_argument("--workload", default="ring_ar_bf16_n8_128MiB", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / verification leg")
    ap.add_argument("--cpu-threads", type=int, default=0, help="threads of the CPU baseline (0 = min(16, cores))")
    ap.add_argument("--shape-sweep", action="store_true",
                    help="ring allreduce bf16 over rank counts x per-rank sizes (both sides of every launch-shape threshold): "
                         "one JSON line with the dominant kernel's fraction of the HBM roofline per point")
    ap.add_argument("--no-via", action="store_true", help="skip the legs that drive the schedule through the primitives")
    ap.add_argument("--no-configs", action="store_true",
                    help="default workload only: leave out the other configurations and the no-reuse leg")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the N ranks are simulated as HBM buffers on it); "
                 "--gpus %d is not supported" % args.gpus)

    import torch
    import __graft_entry__
    __graft_entry__.ensure_built()  # loads what is built; a tree that holds no library yet builds it first
    import hcomm_amd as h

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.Stream(device=dev)  # default priority
    code, thread = h.HcommThreadAllocWithStream(stream.cuda_stream, 32)  # a notify slot per possible peer thread
    h.check(code, "HcommThreadAllocWithStream")
    if args.shape_sweep:
        with torch.cuda.stream(stream):
            out = shape_sweep(args, torch, h, dev, stream, thread)
        h.HcommThreadFreeWithStream([thread])
        print(json.dumps(out))
        return
    with torch.cuda.stream(stream):  # torch's own work (restoring inputs) is ordered with the library's launches
        out = run_workload(args, torch, h, dev, stream, thread)
        if args.workload == "ring_ar_bf16_n8_128MiB" and not args.no_configs:
            out["roofline"]["no_reuse"] = no_reuse_leg(torch, h, dev, stream, thread, max(args.steps, 20))
            rows = []
            for name, steps in CONFIG_LINE:
                sub = argparse.Namespace(workload=name, steps=steps, warmup=2, lowering="both", no_cpu=args.no_cpu,
                                         cpu_threads=args.cpu_threads, cpu_seconds=1.0, no_via=args.no_via)
                r = run_workload(sub, torch, h, dev, stream, thread)
                c = r["config"]
                in_place = c["algorithm"] == "ring_rs_stage"
                footprint = c["ranks"] * c["elements_per_rank"] * {"bf16": 2, "fp16": 2, "fp32": 4, "int32": 4, "int8": 1}[r["dtype"]] * (1 if in_place else 2)
                resident = footprint <= MEMORY_SIDE_CACHE_BYTES
                row = {"workload": name, "ms_per_step": r["ms_per_step"], "ms_per_step_median": r["ms_per_step_median"],
                       "gbs": r["value"],
                       # a workload whose buffers all fit the 256 MiB memory-side cache never goes to HBM after its first
                       # step: its GB/s is cache bandwidth and is not priced against the HBM roofline
                       "frac": None if resident else round(r["value"] / HBM_PEAK_GBS, 4),
                       "footprint_mib": round(footprint / 2 ** 20, 2),
                       "served_from": "memory-side cache (footprint <= 256 MiB)" if resident else "HBM",
                       "launches": r["launches"],
                       "kernel": r["roofline"]["kernel"], "kernel_ms": r["roofline"]["kernel_ms"],
                       "kernel_frac": None if resident else r["roofline"]["frac"], "steps": steps,
                       "traffic": measured_traffic(name, "stepwise"),
                       "algorithmic_bytes_per_launch": r["roofline"]["algorithmic_bytes_per_launch"],
                       "verified": r["verified_bit_exact_vs_oracle"]}
                if r.get("via_primitives"):
                    v = r["via_primitives"]
                    row["via_primitives"] = {"batched_ms": v["batched"]["ms_per_step"],
                                             "host_us_per_batch": v["batched"]["host_us_per_batch"],
                                             "thread_per_rank_ms": v["thread_per_rank"]["ms_per_step"],
                                             "host_thread_per_rank_ms": v["host_thread_per_rank"]["ms_per_step"],
                                             "thread_per_rank_batched_ms": v["thread_per_rank_batched"]["ms_per_step"],
                                             "one_batch_ms": v["one_batch"]["ms_per_step"],
                                             "verified": all(v[m].get("verified") for m in VIA_MODES)}
                for low in ("fused", "fused_keep_inputs"):
                    if r.get(low):
                        row[low + "_ms_per_step"] = r[low]["ms_per_step"]
                        row[low + "_launches"] = r[low]["launches"]
                        row[low + "_moved_gbs"] = round(r[low]["moved_bytes"] / (r[low]["ms_per_step"] * 1e-3) / 1e9, 1)
                rows.append(row)
            # config 4 in full: the 11 message sizes, one fused launch against the step-wise replay
            sweep = mesh_sweep(argparse.Namespace(steps=100, workload="mesh_oneshot_fp16_n8_sweep"), torch, h, dev, stream, thread,
                               8, h.HcommDataType.FP16, 2)
            out["config4_sweep"] = {"what": "mesh one-shot allreduce SUM fp16, 8 ranks: median us of 100 launches timed one by one "
                                            "(fused = one launch for all ranks; stepwise = 8 launches), per-launch us when 100 are "
                                            "queued back to back, GB/s = 72 M / pipelined time; from 1 MiB per rank on the 16 buffers "
                                            "live in the memory-side cache, so those GB/s are not HBM bandwidth",
                                    "launch_floor_us": sweep["launch_floor_us"],
                                    "points": [{"bytes_per_rank": pt["bytes_per_rank"], "fused_us": pt["fused_us"],
                                                "fused_pipelined_us": pt["fused_pipelined_us"], "fused_gbs": pt["fused_gbs"],
                                                "stepwise_us": pt["stepwise_us"], "stepwise_pipelined_us": pt["stepwise_pipelined_us"]}
                                               for pt in sweep["sweep"]]}
            out["configs"] = rows
    h.HcommThreadFreeWithStream([thread])
    print(json.dumps(out))


def run_workload(args, torch, h, dev, stream, thread):
    """One workload: timing of every lowering it has, CPU baseline and verification; returns the result line."""
    import numpy as np
    alg_name, n, count, dtname, opname, dist = WORKLOADS[args.workload]
    DT = {"bf16": h.HcommDataType.BFP16, "fp32": h.HcommDataType.FP32, "fp16": h.HcommDataType.FP16,
          "int32": h.HcommDataType.INT32, "int8": h.HcommDataType.INT8}
    ALG = {"ring_ar": h.Alg.ALLREDUCE_RING, "rhd_ar": h.Alg.ALLREDUCE_RHD, "ring_rs_stage": h.Alg.REDUCE_SCATTER_RING,
           "mesh_oneshot": h.Alg.ALLREDUCE_MESH_ONESHOT, "local_reduce": h.Alg.ALLREDUCE_LOCAL_REDUCE,
           "chunk_mesh": h.Alg.ALLREDUCE_CHUNK_MESH, "nhr": h.Alg.ALLREDUCE_NHR, "nb": h.Alg.ALLREDUCE_NB,
           "local_reduce_rs": h.Alg.REDUCE_SCATTER_LOCAL_REDUCE, "nhr_oneshot": h.Alg.ALLREDUCE_NHR_ONESHOT,
           "doubling": h.Alg.ALLREDUCE_DOUBLING}
    OP = {"sum": h.HcommReduceOp.SUM, "prod": h.HcommReduceOp.PROD, "max": h.HcommReduceOp.MAX,
          "min": h.HcommReduceOp.MIN}
    opbase = alg_name.startswith("opbase_")  # the template inside the op-base loop of its executor
    if opbase:
        alg_name = alg_name[len("opbase_"):]
    hier = None  # (servers, ranks per server): the level-1 template inside the ring executor's three steps
    dbring = False  # the double-ring executor with DMA reduce instead of the single ring on staged buffers
    mesh0 = alg_name.startswith("meshhier")  # the mesh executor's level 0 instead of the ring executor's
    hier_rs = alg_name.startswith("hierrs_") or alg_name.startswith("meshhierrs_")  # the reduce-scatter executors
    ophier = alg_name.startswith("ophier_")  # the order-preserving allreduce executor over two levels
    ophrs = alg_name.startswith("ophierrs_")  # the order-preserving reduce-scatter executor over two levels
    if alg_name.startswith("hier") or alg_name.startswith("dbring_") or mesh0 or ophier or ophrs:
        dbring = alg_name.startswith("dbring_")
        alg_name, hier, n = alg_name.split("_", 1)[1], n, n[0] * n[1]
    dbhrs = None  # (pods, servers per pod, ranks per server) of the double-ring reduce-scatter executor over several servers
    if alg_name == "doublering_hier_rs":
        dbhrs = n if len(n) == 3 else (1,) + tuple(n)
        n = dbhrs[0] * dbhrs[1] * dbhrs[2]
    ccl_bytes = 200 << 20  # HCCL_CCL_COMM_DEFAULT_BUFFER_SIZE, src/legacy/ascend910/pub_inc/externalinput_pub.h:37
    # one-server executors on user memory (DMA reduce)
    plant = alg_name in ("order_preserved_rs", "doublering_rs", "doublering_hier_rs", "order_preserved_ar", "order_preserved_small")
    opsmall = alg_name == "order_preserved_small"
    opar = alg_name == "order_preserved_ar"
    # the order-preserving executors also have a single-launch lowering
    opfused = alg_name in ("order_preserved_ar", "order_preserved_rs") or ophier or ophrs
    dbrs = alg_name == "doublering_rs"
    dt, alg, op = DT[dtname], (None if plant else ALG[alg_name]), OP[opname]
    unit = h.DTYPE_SIZE[dt]
    in_place = alg_name == "ring_rs_stage" and not hier

    if count is None:
        return mesh_sweep(args, torch, h, dev, stream, thread, n, dt, unit)

    nbytes = count * unit
    in_count = n * count if (alg_name in ("local_reduce_rs", "order_preserved_rs", "doublering_rs", "doublering_hier_rs",
                                          "order_preserved_small")
                            or hier_rs or ophrs) else count
    pristine = make_inputs(torch, dev, n, in_count, "fp32prod" if opname == "prod" else dtname)
    d_in = [torch.empty(in_count * unit, dtype=torch.uint8, device=dev) for _ in range(n)]
    d_out = None if in_place else [torch.empty(nbytes, dtype=torch.uint8, device=dev) for _ in range(n)]

    def restore():
        """Inputs as generated, outputs zero; queued on the stream the library launches on (no host wait)."""
        for r in range(n):
            d_in[r].copy_(pristine[r])
        if d_out is not None:
            for r in range(n):
                d_out[r].zero_()

    in_ptrs = [t.data_ptr() for t in d_in]
    out_ptrs = None if in_place else [t.data_ptr() for t in d_out]
    scratch_bytes = 0 if plant else h.scratch_bytes(alg, n, count, dt)
    d_ccl = None
    if opbase or dbring or plant or hier_rs or ophier or ophrs:
        d_ccl = [[torch.zeros(ccl_bytes, dtype=torch.uint8, device=dev) for _ in range(n)] for _ in range(2)]
        if args.lowering == "both" and not opfused:
            args.lowering = "stepwise"
    if (hier and not opfused) or (plant and not opfused):
        args.lowering = "stepwise"  # composed from the step lists of its levels
    d_scr = [torch.zeros(scratch_bytes, dtype=torch.uint8, device=dev) for _ in range(n)] if scratch_bytes else None
    scr_ptrs = [t.data_ptr() for t in d_scr] if d_scr else None
    kname = {h.Kernel.REDUCE2: "k_reduce2", h.Kernel.CHAIN: "k_fold_chain", h.Kernel.TREE: "k_fold_tree",
             h.Kernel.COPY: "k_copy", h.Kernel.BYTEWISE: "k_bytewise"}

    def make_plan(low):
        if hier_rs:
            return h.HierReduceScatterPlan(alg, hier[0], hier[1], in_ptrs, out_ptrs, [t.data_ptr() for t in d_ccl[0]],
                                           [t.data_ptr() for t in d_ccl[1]], ccl_bytes, count, dt, op, mesh=mesh0)
        if dbhrs:
            return h.DoubleRingHierReduceScatterPlan(h.Alg.REDUCE_SCATTER_RING, dbhrs[1], dbhrs[2], in_ptrs, out_ptrs,
                                                     [t.data_ptr() for t in d_ccl[0]], ccl_bytes, count, dt, op, n_pods=dbhrs[0])
        if dbrs:
            return h.DoubleRingReduceScatterPlan(in_ptrs, out_ptrs, [t.data_ptr() for t in d_ccl[0]], ccl_bytes, count, dt, op)
        if opfused and low == h.Lowering.FUSED:  # one launch on the user buffers, no CCL buffer
            return h.OrderPreservedFusedPlan(opar or ophier, in_ptrs, out_ptrs, count, dt, op, n_servers=hier[0] if hier else 1)
        if opsmall:
            return h.OrderPreservedSmallPlan(in_ptrs, out_ptrs, [t.data_ptr() for t in d_ccl[1]], ccl_bytes, count, dt, op)
        if opar:
            return h.OrderPreservedAllReducePlan(in_ptrs, out_ptrs, [t.data_ptr() for t in d_ccl[0]],
                                                 [t.data_ptr() for t in d_ccl[1]], ccl_bytes, count, dt, op)
        if plant:
            return h.OrderPreservedPlan(in_ptrs, out_ptrs, [t.data_ptr() for t in d_ccl[1]], ccl_bytes, count, dt, op)
        if ophrs:
            return h.OrderPreservedHierReduceScatterPlan(hier[0], hier[1], in_ptrs, out_ptrs, [t.data_ptr() for t in d_ccl[1]],
                                                         ccl_bytes, count, dt, op)
        if ophier:
            return h.OrderPreservedHierAllReducePlan(alg, hier[0], hier[1], in_ptrs, out_ptrs, [t.data_ptr() for t in d_ccl[0]],
                                                     [t.data_ptr() for t in d_ccl[1]], ccl_bytes, count, dt, op)
        if dbring:
            return h.DoubleRingPlan(alg, hier[0], hier[1], in_ptrs, out_ptrs, [t.data_ptr() for t in d_ccl[0]],
                                    [t.data_ptr() for t in d_ccl[1]], ccl_bytes, count, dt, op)
        if hier:
            return h.HierPlan(alg, hier[0], hier[1], in_ptrs, out_ptrs, count, dt, op, mesh=mesh0)
        if opbase:
            return h.OpBasePlan(alg, low, in_ptrs, out_ptrs, [t.data_ptr() for t in d_ccl[0]],
                                [t.data_ptr() for t in d_ccl[1]], ccl_bytes, count, dt, op, scr_ptrs)
        return h.Plan(alg, low, in_ptrs, out_ptrs, count, dt, op, 0, scr_ptrs)

    def kernel_name(rec):
        """The kernel a launch record names, as the profiler shows it (template arguments as type and op names)."""
        copy = rec.op == 255
        if rec.kind == h.Kernel.BYTEWISE:
            return "k_bytewise<copy>" if copy else "k_bytewise<%s,%s>" % (dtname, opname.upper())
        base = kname[rec.kind]
        if rec.rows:  # the variants that read every address in one round
            base += "_rows" if rec.kind in (h.Kernel.COPY, h.Kernel.REDUCE2) else "_direct"
        return base if copy else "%s<%s,%s>" % (base, dtname, opname.upper())

    lowerings = ["stepwise", "fused"] if args.lowering == "both" else [args.lowering]
    # a template on the rank buffers themselves also has the fused launches without their stores into the inputs
    plain_plan = not (hier_rs or dbrs or opfused or opsmall or opar or plant or ophrs or ophier or dbring or hier or opbase)
    if args.lowering == "both" and plain_plan and not in_place:
        lowerings.append("fused_keep_inputs")
    lowering_of = {"stepwise": h.Lowering.STEPWISE, "fused": h.Lowering.FUSED,
                   "fused_keep_inputs": h.Lowering.FUSED_KEEP_INPUTS}
    results = {}
    for name in lowerings:
        low = lowering_of[name]
        try:
            plan = make_plan(low)
        except h.HcommError as e:  # e.g. the single-launch reduce-scatter needs blocks of whole 16 bytes
            if name != "stepwise" and e.code == h.HcclResult.E_NOT_SUPPORT:
                continue
            raise
        launches = plan.launches()
        for _ in range(args.warmup):
            restore()
            h.check(plan.run(thread), "HcommGfxPlanRun")
        stream.synchronize()
        # EXACTLY args.steps steps, every one of them on the inputs as generated: the inputs are restored before
        # each step (outside the timed events), and a step is timed by a pair of HIP events on the launch stream
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        for a, b in ev:
            restore()
            a.record(stream)
            h.check(plan.run(thread), "HcommGfxPlanRun")
            b.record(stream)
        stream.synchronize()
        torch.cuda.synchronize()
        per_step = sorted(a.elapsed_time(b) for a, b in ev)
        ms_step = sum(per_step) / args.steps
        # for comparison: the same number of steps queued back to back with no restore in between, timed by the
        # host clock (from the second step on they run on what the step before left in the buffers)
        restore()
        stream.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            h.check(plan.run(thread), "HcommGfxPlanRun")
        stream.synchronize()
        ms_back_to_back = (time.perf_counter() - t0) * 1e3 / args.steps

        # dominant kernel = the kind with the most bytes; its first contiguous run of launches is timed as a
        # group with HIP events recorded on the stream the kernels run on, again on restored inputs
        # (the kernel for unaligned operands comes as a copy and as a reduce: op 255 marks the copies)
        kkey = lambda r: (r.kind, r.op == 255)
        by_kind = {}
        for r in launches:
            by_kind[kkey(r)] = by_kind.get(kkey(r), 0) + r.bytes * (2 if r.op == 255 else 3)
        dom_key = max(by_kind, key=by_kind.get)
        dom_kind, dom_is_copy = dom_key
        first = [i for i, r in enumerate(launches) if kkey(r) == dom_key][0]
        cnt = 1
        while first + cnt < len(launches) and kkey(launches[first + cnt]) == dom_key:
            cnt += 1
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        for a, b in ev:
            restore()
            if first:
                h.check(plan.run_range(thread, 0, first), "run_range")
            a.record(stream)
            h.check(plan.run_range(thread, first, cnt), "run_range")
            b.record(stream)
            rest = plan.info.launches - first - cnt
            if rest:
                h.check(plan.run_range(thread, first + cnt, rest), "run_range")
        stream.synchronize()
        dom_ms = sum(a.elapsed_time(b) for a, b in ev) / (args.steps * cnt)
        if name == "stepwise":
            # average launch of the run: 3 x (bytes it writes) for a reduce step of all ranks, 2 x for a copy step
            per_byte = 2 if dom_is_copy else 3
            dom_bytes = sum(launches[i].bytes for i in range(first, first + cnt)) * per_byte // cnt
            dom_moved = dom_bytes
        else:
            # the launches of the run (one, or one per group of ranks) are the whole collective: per-launch shares
            dom_bytes = plan.info.algorithmicBytes // cnt
            dom_moved = plan.info.movedBytes // cnt
        results[name] = {
            "ms_per_step": ms_step,
            "ms_per_step_min": per_step[0],
            "ms_per_step_median": per_step[len(per_step) // 2],
            "ms_per_step_back_to_back": ms_back_to_back,
            "gbs": plan.info.algorithmicBytes / (ms_step * 1e-3) / 1e9,
            "launches": plan.info.launches,
            "algorithmic_bytes": plan.info.algorithmicBytes,
            "moved_bytes": plan.info.movedBytes,
            "kernel": kernel_name(launches[first]),
            "kernel_variant": ("rows" if launches[first].rows else "one-dimensional") + (", streaming" if launches[first].streaming else ""),
            "kernel_ms": dom_ms,
            "kernel_alg_bytes": dom_bytes,
            "kernel_gbs": dom_bytes / (dom_ms * 1e-3) / 1e9,
            "kernel_moved_gbs": dom_moved / (dom_ms * 1e-3) / 1e9,
        }
        plan.destroy()

    via, via_run, via_done = None, None, None
    if plain_plan and "stepwise" in results and not getattr(args, "no_via", False):
        via, via_run, via_done = via_primitives_leg(args, torch, h, stream, thread, alg, n, count, dt, op, in_ptrs, out_ptrs, scr_ptrs, restore,
                                 results["stepwise"])

    # The headline is the step-wise replay: every launch is one schedule step of two-input reduces / copies, so
    # the bytes it moves ARE the algorithmic bytes.
    best = "stepwise" if "stepwise" in results else lowerings[0]
    res = results[best]

    cpu = None
    verified = None
    if not args.no_cpu:
        import oracle
        threads = args.cpu_threads or min(16, os.cpu_count() or 1)
        odt = {"bf16": oracle.BF16, "fp32": oracle.F32, "fp16": oracle.F16, "int32": oracle.I32,
               "int8": oracle.I8}[dtname]
        oalg = {"ring_ar": oracle.ALG_ALLREDUCE_RING, "rhd_ar": oracle.ALG_ALLREDUCE_RHD,
                "ring_rs_stage": oracle.ALG_RS_RING_STAGE, "mesh_oneshot": oracle.ALG_ALLREDUCE_MESH_ONESHOT,
                "local_reduce": oracle.ALG_ALLREDUCE_LOCAL_REDUCE, "chunk_mesh": oracle.ALG_ALLREDUCE_CHUNK_MESH,
                "nhr": oracle.ALG_ALLREDUCE_NHR, "nb": oracle.ALG_ALLREDUCE_NB,
                "local_reduce_rs": oracle.ALG_RS_LOCAL_REDUCE, "nhr_oneshot": oracle.ALG_ALLREDUCE_NHR_ONESHOT,
                "doubling": oracle.ALG_ALLREDUCE_DOUBLING,
                "order_preserved_rs": None, "doublering_rs": None, "doublering_hier_rs": None, "order_preserved_ar": None,
                "order_preserved_small": None}[alg_name]
        oop = {"sum": oracle.SUM, "prod": oracle.PROD, "max": oracle.MAX, "min": oracle.MIN}[opname]
        npdt = oracle.NP_STORAGE[odt]
        host_in = [p.cpu().numpy().view(npdt).copy() for p in pristine]
        host_out = [np.zeros(count if not in_place else 1, npdt) for _ in range(n)]
        oracle.lib().orc_set_threads(threads)
        host_scr = [np.zeros(scratch_bytes, np.uint8) for _ in range(n)] if scratch_bytes else None
        if hier_rs:
            alg_bytes = sum(o[8] * (3 if o[1] else 2)
                            for o in oracle.trace_hier_rs(oalg, hier[0], hier[1], count, ccl_bytes, odt, mesh=mesh0))
        elif dbhrs:
            alg_bytes = sum(o[8] * (3 if o[1] else 2) for o in oracle.trace_dbring_rs_servers(
                oracle.ALG_RS_RING_STAGE, dbhrs[1], dbhrs[2], count, ccl_bytes, odt, n_pods=dbhrs[0]))
        elif dbrs:
            alg_bytes = sum(o[8] * (3 if o[1] else 2) for o in oracle.trace_dbring_rs(n, count, ccl_bytes, odt))
        elif opsmall:
            alg_bytes = sum(o[8] * (3 if o[1] else 2) for o in oracle.trace_order_preserved_small(n, count, ccl_bytes, odt))
        elif opar:
            alg_bytes = sum(o[8] * (3 if o[1] else 2) for o in oracle.trace_order_preserved_ar(n, count, ccl_bytes, odt))
        elif plant:
            alg_bytes = sum(o[8] * (3 if o[1] else 2) for o in oracle.trace_order_preserved(n, count, ccl_bytes, odt))
        elif ophrs:
            alg_bytes = sum(o[8] * (3 if o[1] else 2)
                            for o in oracle.trace_order_preserved_rs2(hier[0], hier[1], count, ccl_bytes, odt))
        elif ophier:
            alg_bytes = sum(o[8] * (3 if o[1] else 2)
                            for o in oracle.trace_order_preserved_ar2(oalg, hier[0], hier[1], count, ccl_bytes, odt))
        elif dbring:
            alg_bytes = sum(o[8] * (3 if o[1] else 2)
                            for o in oracle.trace_dbring(oalg, hier[0], hier[1], count, ccl_bytes, odt))
        elif hier:
            alg_bytes = sum(o[8] * (3 if o[1] else 2)
                            for o in oracle.trace_hier(oalg, hier[0], hier[1], count, odt, mesh=mesh0))
        else:
            alg_bytes = (oracle.algorithmic_bytes_opbase(oalg, n, count, ccl_bytes, odt) if opbase
                         else oracle.algorithmic_bytes(oalg, n, count, odt))
        host_ccl = ([[np.zeros(ccl_bytes, np.uint8) for _ in range(n)] for _ in range(2)]
                    if (opbase or dbring or plant or hier_rs or ophier or ophrs) else None)

        def cpu_run(ins, outs):
            if hier_rs:
                oracle.run_hier_rs(oalg, hier[0], hier[1], ins, outs, host_ccl[0], host_ccl[1], count, ccl_bytes, odt, oop,
                                   mesh=mesh0)
            elif dbhrs:
                oracle.run_dbring_rs_servers(oracle.ALG_RS_RING_STAGE, dbhrs[1], dbhrs[2], ins, outs, host_ccl[0], count,
                                             ccl_bytes, odt, oop, n_pods=dbhrs[0])
            elif dbrs:
                oracle.run_dbring_rs(ins, outs, host_ccl[0], count, ccl_bytes, odt, oop)
            elif opsmall:
                oracle.run_order_preserved_small(ins, outs, host_ccl[0], host_ccl[1], count, ccl_bytes, odt, oop)
            elif opar:
                oracle.run_order_preserved_ar(ins, outs, host_ccl[0], host_ccl[1], count, ccl_bytes, odt, oop)
            elif plant:
                oracle.run_order_preserved(ins, outs, host_ccl[0], host_ccl[1], count, ccl_bytes, odt, oop)
            elif ophrs:
                oracle.run_order_preserved_rs2(hier[0], hier[1], ins, outs, host_ccl[0], host_ccl[1], count, ccl_bytes, odt, oop)
            elif ophier:
                oracle.run_order_preserved_ar2(oalg, hier[0], hier[1], ins, outs, host_ccl[0], host_ccl[1], count, ccl_bytes,
                                               odt, oop)
            elif dbring:
                oracle.run_dbring(oalg, hier[0], hier[1], ins, outs, host_ccl[0], host_ccl[1], count, ccl_bytes, odt, oop)
            elif hier:
                oracle.run_hier(oalg, hier[0], hier[1], ins, outs, count, odt, oop, mesh=mesh0)
            elif opbase:
                oracle.run_opbase(oalg, ins, outs, host_ccl[0], host_ccl[1], count, ccl_bytes, odt, oop, scratch=host_scr)
            else:
                oracle.run(oalg, ins, outs, count, odt, oop, scratch=host_scr)

        passes, cpu_s = 0, 0.0
        cpu_budget = getattr(args, "cpu_seconds", 8.0)
        while passes < 1 or (cpu_s < cpu_budget and passes < 64):
            work_in = [x.copy() for x in host_in]  # every pass starts from the pristine inputs (copy not timed)
            t0 = time.perf_counter()
            cpu_run(work_in, host_out)
            cpu_s += time.perf_counter() - t0
            passes += 1
        host_in = work_in
        # the same schedule on ONE thread (the scalar loop shape of the reference's CPU witnesses), one pass
        one_s = None
        if cpu_budget >= 8.0:
            oracle.lib().orc_set_threads(1)
            one_in = [p.cpu().numpy().view(npdt).copy() for p in pristine]
            one_out = [np.zeros(count if not in_place else 1, npdt) for _ in range(n)]
            t0 = time.perf_counter()
            cpu_run(one_in, one_out)
            one_s = time.perf_counter() - t0
            del one_in, one_out
        model = "unknown"
        try:
            # the first processor's entry: model name plus what identifies the part when a hypervisor blanks the name
            info = {}
            with open("/proc/cpuinfo") as f:
                for l in f:
                    if ":" not in l:
                        if info:
                            break
                        continue
                    k, v = l.split(":", 1)
                    info.setdefault(k.strip(), v.strip())
            model = "%s (vendor %s, family %s, model %s, stepping %s, %s MHz, cache %s)" % (
                info.get("model name", "?"), info.get("vendor_id", "?"), info.get("cpu family", "?"), info.get("model", "?"),
                info.get("stepping", "?"), info.get("cpu MHz", "?"), info.get("cache size", "?"))
        except Exception:
            pass
        cpu = {"value": round(alg_bytes * passes / cpu_s / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
               "sample": "the full workload, %d passes, %.2f s of CPU work in total; OpenMP static over elements"
                         % (passes, cpu_s),
               "single_thread_value": round(alg_bytes / one_s / 1e9, 2) if one_s else None, "cpu_model": model,
               "host_cores": os.cpu_count()}
        # the reference's own CPU reduce loop (VirtualRunTime::MemReduceSum, test/hccl_vm/src/plugin/runner/
        # runner_utils/hccl_task_reduce_process.cc:57-84, compiled from where it lies into oracle/_ref) on one
        # thread, for the element types it has (no bf16 there): dst = dst + src over a bounded sample, 3 bytes
        # of traffic per byte of dst
        if oracle.have_ref() and cpu_budget >= 8.0:
            R = oracle.ref()
            rng = np.random.default_rng(7)
            witness = {}
            for rname, rdt, elems in (("fp32", oracle.F32, 1 << 24), ("fp16", oracle.F16, 1 << 22), ("int32", oracle.I32, 1 << 24)):
                if rdt == oracle.F16:
                    d_ = rng.uniform(-1, 1, elems).astype(np.float16).view(np.uint16)
                    s_ = rng.uniform(-1, 1, elems).astype(np.float16).view(np.uint16)
                elif rdt == oracle.F32:
                    d_, s_ = (rng.uniform(-1, 1, elems).astype(np.float32) for _ in range(2))
                else:
                    d_, s_ = (rng.integers(-1 << 20, 1 << 20, elems).astype(np.int32) for _ in range(2))
                reps, t_ref = 0, 0.0
                while reps < 1 or (t_ref < 1.0 and reps < 64):
                    t0 = time.perf_counter()
                    R.ref_mem_reduce_sum(s_.ctypes.data, d_.ctypes.data, d_.nbytes, rdt)
                    t_ref += time.perf_counter() - t0
                    reps += 1
                witness[rname] = round(3.0 * d_.nbytes * reps / t_ref / 1e9, 2)
            cpu["reference_reduce"] = {"kind": "reference", "function": "VirtualRunTime::MemReduceSum", "cores": 1,
                                       "unit": "GB/s", "value_by_dtype": witness,
                                       "sample": "dst += src over 2^24 fp32 / int32 and 2^22 fp16 elements, >= 1 s each"}
        # verification: one GPU pass per lowering from pristine inputs must equal the oracle bit for bit
        verified = True
        for name in lowerings:
            if name not in results:
                continue
            low = lowering_of[name]
            plan = make_plan(low)
            restore()
            h.check(plan.run(thread), "HcommGfxPlanRun")
            stream.synchronize()
            torch.cuda.synchronize()
            for r in range(n):
                if name == "fused_keep_inputs":  # the inputs as they were, not as the replay leaves them
                    ok = bool(torch.equal(d_in[r], pristine[r]))
                else:
                    ok = np.array_equal(d_in[r].cpu().numpy(), host_in[r].view(np.uint8))
                if not in_place:
                    ok = ok and np.array_equal(d_out[r].cpu().numpy(), host_out[r].view(np.uint8))
                if (opbase or dbring or plant or hier_rs or ophier or ophrs) and not (opfused and name == "fused"):  # what the last chunk left in the CCL buffers
                    ok = ok and np.array_equal(d_ccl[0][r].cpu().numpy(), host_ccl[0][r])
                    ok = ok and np.array_equal(d_ccl[1][r].cpu().numpy(), host_ccl[1][r])
                verified = verified and bool(ok)
            plan.destroy()
        if via is not None:
            # the same schedule driven through the primitives must leave the same bits
            for mode in VIA_MODES:
                restore()
                if d_scr:
                    for t in d_scr:
                        t.zero_()
                via_run[mode]()
                stream.synchronize()
                torch.cuda.synchronize()
                ok = True
                for r in range(n):
                    ok = ok and np.array_equal(d_in[r].cpu().numpy(), host_in[r].view(np.uint8))
                    if not in_place:
                        ok = ok and np.array_equal(d_out[r].cpu().numpy(), host_out[r].view(np.uint8))
                via[mode]["verified"] = bool(ok)
                verified = verified and bool(ok)
    if via_done is not None:
        via_done()

    metric = "HBM GB/s (% of peak) for simulated 8-rank bf16 ring allreduce, 128MiB/rank"
    if args.workload != "ring_ar_bf16_n8_128MiB":
        metric = "HBM GB/s (%% of peak) for simulated %d-rank %s %s %s" % (n, dtname, ("order-preserving two-level " if (ophier or ophrs) else "double-ring " if dbring else "mesh three-step " if mesh0 else "three-step " if hier else "") + ("reduce-scatter" if ophrs else "allreduce" if ophier else alg_name), opname)
    out = {
        "metric": metric,
        "value": round(res["gbs"], 2),
        "unit": "GB/s",
        "pct_of_peak": round(100.0 * res["gbs"] / HBM_PEAK_GBS, 2),
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(res["ms_per_step"], 5),
        "ms_per_step_min": round(res["ms_per_step_min"], 5),
        "ms_per_step_median": round(res["ms_per_step_median"], 5),
        "ms_per_step_back_to_back": round(res["ms_per_step_back_to_back"], 5),
        "timing": "every step runs on the inputs as generated (restored before it, outside the timed region) and is "
                  "timed by a pair of HIP events on the launch stream; ms_per_step is the mean over the steps; "
                  "ms_per_step_back_to_back is the host clock over the same number of steps queued without restores",
        "launches": res["launches"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtname,
        "data": "synthetic",
        "config": {"workload": args.workload, "ranks": n, "elements_per_rank": count, "op": opname,
                   "algorithm": ("order_preserved_rs" if ophrs else "order_preserved_ar" if ophier else alg_name),
                   "values": dist, "seed": "torch generator on the GPU, 1234 + rank", "lowering": best,
                   **({"op_base_loop": True, "ccl_buffer_bytes": ccl_bytes} if opbase else {}),
                   **({"servers": hier[0], "ranks_per_server": hier[1], "level1_algorithm": ("plant + fold in server order (combine template)" if ophrs else
                                            "plant + fold in server order (combine template), %s all-gather" % alg_name
                                            if ophier else alg_name),
                       "level0_algorithm": ("plant + fold in device order (user memory read directly)" if ophrs else
                                            "plant + fold in device order, mesh all-gather (user memory read directly)" if ophier else
                                            "double-ring reduce-scatter + all-gather on user memory (DMA reduce)"
                                            if dbring else "multi-stream mesh reduce-scatter + mesh all-gather" if mesh0
                                            else "ring reduce-scatter + ring all-gather")} if hier else {}),
                   **({"ccl_buffer_bytes": ccl_bytes} if (dbring or plant or hier_rs or ophier or ophrs) else {})},
        "roofline": {"bound": "hbm", "achieved": round(res["kernel_gbs"], 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(res["kernel_gbs"] / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic(args.workload, best),
                     "traffic_is": "L2 <-> fabric bytes (FETCH_SIZE / WRITE_SIZE count below the L2): equal to the "
                                   "algorithmic bytes means no re-reads and no write amplification; how many of them "
                                   "the memory-side cache served instead of HBM these counters cannot tell",
                     "kernel": res["kernel"], "kernel_variant": res["kernel_variant"], "kernel_ms": round(res["kernel_ms"], 5),
                     "algorithmic_bytes_per_launch": res["kernel_alg_bytes"]},
        "cpu_baseline": cpu,
        "verified_bit_exact_vs_oracle": verified,
        "via_primitives": via,
        "fused": ({kk: (round(vv, 5) if isinstance(vv, float) else vv) for kk, vv in results["fused"].items()}
                  if "fused" in results and best != "fused" else None),
        "fused_keep_inputs": ({kk: (round(vv, 5) if isinstance(vv, float) else vv)
                               for kk, vv in results["fused_keep_inputs"].items()}
                              if "fused_keep_inputs" in results else None),
    }
    return out


VIA_MODES = ("batched", "thread_per_rank", "host_thread_per_rank", "thread_per_rank_batched", "one_batch")


def via_primitives_leg(args, torch, h, stream, thread, alg, n, count, dt, op, in_ptrs, out_ptrs, scr_ptrs, restore, plan_res):
    """The same schedule driven through the reference's own boundary by a caller that knows nothing but the
    primitives (hcomm_amd/csrc/hg_caller.c):
      batched          per schedule step HcommBatchModeStart, every rank's HcommLocalCopy/ReduceOnThread call,
                       HcommBatchModeEnd, all on the thread the plans run on (cpu_primitives_c_adpt.cc:58-130,
                       launch_context.cc:139-174): the coalescing a plan does once at creation happens inside every End;
      thread_per_rank  rank r's calls on a thread (stream) of its own, nothing batched, notifies between the steps the
                       way the templates post and wait (reduce_scatter_ring.cc:211-217,254-272); thread 0 is the stream
                       the events are recorded on, the others fork from and join it; ONE host thread issues everything;
      host_thread_per_rank  the same with a host thread per rank issuing that rank's calls (the ranks of the reference
                       are processes of their own);
      thread_per_rank_batched  the calls of thread_per_rank, posts and waits included, between ONE HcommBatchModeStart /
                       End pair - the whole collective as one batch over all its threads, what the reference submits as
                       one task graph (launch_context.cc:16-44); HcommBatchModeEnd resolves the notifies on the host;
      one_batch        every call of the collective between ONE Start / End pair on the one thread.
    Timed like the plans: inputs restored before every step, a pair of HIP events around it."""
    from hcomm_amd import caller
    ops = h.schedule_emit(alg, n, count, dt)
    bufs = {0: in_ptrs}
    if out_ptrs is not None:
        bufs[1] = out_ptrs
    if scr_ptrs:
        bufs[2] = scr_ptrs
    replay = caller.Replay(ops, bufs, dt, op)
    others = []
    if n > 1:
        code, others = h.HcommThreadAlloc(h.CommEngine.CPU_TS, n - 1, 32)
        h.check(code, "HcommThreadAlloc")
    threads = [thread] + others
    last = {}

    def run_batched():
        code, st = replay.run_batched(thread)
        h.check(code, "replay through HcommBatchModeStart/End")
        last["batched"] = st

    def run_threads():
        code, st = replay.run_on_threads(threads)
        h.check(code, "replay on one thread per rank")
        last["thread_per_rank"] = st

    def run_host_threads():
        code, st = replay.run_on_host_threads(threads)
        h.check(code, "replay on one thread and one host thread per rank")
        last["host_thread_per_rank"] = st

    def run_one_batch():
        code, st = replay.run_one_batch(thread)
        h.check(code, "replay as one batch on one thread")
        last["one_batch"] = st

    def run_threads_batched():
        code, st = replay.run_on_threads_batched(threads)
        h.check(code, "replay on one thread per rank inside one batch")
        last["thread_per_rank_batched"] = st

    out = {"what": "the schedule's op list (HcommGfxScheduleEmit) issued call by call through the reference's primitives "
                   "by hcomm_amd/csrc/hg_caller.c, which binds the library with dlsym",
           "plan_ms_per_step": round(plan_res["ms_per_step"], 5)}
    for mode, run in (("batched", run_batched), ("thread_per_rank", run_threads), ("host_thread_per_rank", run_host_threads),
                      ("thread_per_rank_batched", run_threads_batched), ("one_batch", run_one_batch)):
        for _ in range(args.warmup):
            restore()
            run()
        stream.synchronize()
        h.HcommGfxThreadSynchronize(thread)
        h.HcommGfxLaunchLogClear(thread)
        for t in others:
            h.HcommGfxLaunchLogClear(t)
        restore()
        run()
        stream.synchronize()
        launches = sum(len(h.launch_log(t)) for t in threads)
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        host_us, end_us, notify_us = 0.0, 0.0, 0.0
        for a, b in ev:
            restore()
            a.record(stream)
            run()
            b.record(stream)
            st = last[mode]
            host_us += st.host_us
            end_us += st.host_us_end
            notify_us += st.host_us_notify
        stream.synchronize()
        torch.cuda.synchronize()
        per = sorted(a.elapsed_time(b) for a, b in ev)
        ms = sum(per) / len(per)
        st = last[mode]
        row = {"ms_per_step": round(ms, 5), "ms_per_step_min": round(per[0], 5),
               "ms_per_step_median": round(per[len(per) // 2], 5),
               "vs_plan": round(ms / plan_res["ms_per_step"], 4), "launches": launches, "calls": st.calls,
               "host_us_per_step": round(host_us / args.steps, 2)}
        if mode == "one_batch":
            row["batches"] = 1
            row["host_us_in_end"] = round(end_us / args.steps, 2)
        elif mode == "batched":
            row["batches"] = st.batches
            row["host_us_per_batch"] = round(host_us / args.steps / max(st.batches, 1), 2)
            row["host_us_in_end_per_batch"] = round(end_us / args.steps / max(st.batches, 1), 2)
        else:
            row["threads"] = len(threads)
            row["notify_pairs"] = st.notifies
            row["host_us_in_notifies"] = round(notify_us / args.steps, 2)
            if mode == "host_thread_per_rank":
                row["host_threads"] = len(threads)
                row["host_us_in_notifies"] = round(notify_us / args.steps / len(threads), 2)  # per host thread
                row["host_us_slowest_thread"] = round(st.host_us_end_max, 2)
            if mode == "thread_per_rank_batched":
                row["batches"] = 1
                row["host_us_in_end"] = round(end_us / args.steps, 2)
        out[mode] = row
        h.HcommGfxLaunchLogClear(thread)

    def done():
        caller.pool_shutdown()
        for t in others:
            h.HcommGfxThreadSynchronize(t)
        if others:
            h.HcommThreadFree(others)

    return out, {"batched": run_batched, "thread_per_rank": run_threads, "host_thread_per_rank": run_host_threads,
                 "thread_per_rank_batched": run_threads_batched, "one_batch": run_one_batch}, done


def shape_sweep(args, torch, h, dev, stream, thread):
    """Ring allreduce SUM bf16, step-wise, over rank counts and per-rank sizes chosen on both sides of the sizes at which
    a launch changes shape (a reduce launch of a ring step writes one slice per rank = the per-rank size: streaming from
    64 MiB on; a copy streams from 256 MiB on).  Per point: time, algorithmic GB/s, and the reduce kernel's fraction of
    the HBM roofline from HIP events around its launches."""
    points = []
    for n in (4, 8, 16, 32):
        for mib in (32, 63, 65, 128, 255, 257, 512):
            name = "ring_ar_bf16_n%d_%dMiB" % (n, mib)
            WORKLOADS[name] = ("ring_ar", n, mib << 19, "bf16", "sum", "normal(0,1)*1e-3")
            sub = argparse.Namespace(workload=name, steps=max(5, min(args.steps, 10)), warmup=2, lowering="stepwise", no_cpu=True,
                                     cpu_threads=0, no_via=True)
            r = run_workload(sub, torch, h, dev, stream, thread)
            footprint = 2 * n * (mib << 20)
            points.append({"ranks": n, "mib_per_rank": mib, "ms_per_step": r["ms_per_step"], "gbs": r["value"],
                           "frac": round(r["value"] / HBM_PEAK_GBS, 4), "kernel": r["roofline"]["kernel"],
                           "kernel_variant": r["roofline"]["kernel_variant"], "kernel_us": round(r["roofline"]["kernel_ms"] * 1e3, 2),
                           "kernel_frac": r["roofline"]["frac"], "footprint_mib": footprint >> 20})
            torch.cuda.empty_cache()
    return {"metric": "ring allreduce SUM bf16, step-wise: fraction of the HBM roofline over rank counts and per-rank sizes",
            "unit": "fraction of 8 TB/s", "n_gpus": 1, "points": points}


def no_reuse_leg(torch, h, dev, stream, thread, reps):
    """The two-input reduce on operands that nothing touched recently, through the reference's own primitive API:
    one batch of HcommLocalReduceOnThread calls = one k_reduce2_rows<bf16,SUM> launch (equally long segments: the
    two-dimensional grid), rotated over buffer sets so that a
    launch finds nothing of its operands in the 256 MB memory-side cache.
      ring_step_shape   8 segments of 16 MiB (the headline's launch: 128 MiB written), 12 sets of 256 MiB -> 3 GiB
                        between two uses
      streaming_shape   16 segments of 64 MiB (1 GiB written: the first halving step of the 16-rank
                        recursive-halving allreduce), 3 sets of 2 GiB"""
    import ctypes
    hip = ctypes.CDLL(os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so"))  # the runtime torch has loaded
    hip.hipMemcpyAsync.restype = ctypes.c_int
    hip.hipMemcpyAsync.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p]
    out = {}
    for key, nseg, seg_bytes, sets in (("ring_step_shape", 8, 16 << 20, 12), ("streaming_shape", 16, 64 << 20, 3)):
        gen = torch.Generator(device=dev)
        gen.manual_seed(4321)
        elems = seg_bytes // 2
        bufs = []
        for _ in range(sets):
            pairs = []
            for _ in range(nseg):
                d = (torch.randn(elems, generator=gen, device=dev, dtype=torch.float32) * 1e-3).to(torch.bfloat16)
                p = (torch.randn(elems, generator=gen, device=dev, dtype=torch.float32) * 1e-3).to(torch.bfloat16)
                pairs.append((d, p))
            bufs.append(pairs)

        def launch(k):
            h.check(h.HcommBatchModeStart(b"no_reuse"), "HcommBatchModeStart")
            for d, p in bufs[k % sets]:
                h.check(h.HcommLocalReduceOnThread(thread, d.data_ptr(), p.data_ptr(), elems, h.HcommDataType.BFP16,
                                                   h.HcommReduceOp.SUM), "HcommLocalReduceOnThread")
            h.check(h.HcommBatchModeEnd(b"no_reuse"), "HcommBatchModeEnd")

        def timed(fn, bytes_per_launch, kernel):
            for k in range(sets):
                fn(k)
            stream.synchronize()
            ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
            for k, (a, b) in enumerate(ev):
                a.record(stream)
                fn(k)
                b.record(stream)
            stream.synchronize()
            ms = sum(a.elapsed_time(b) for a, b in ev) / reps
            return {"kernel": kernel, "kernel_ms": round(ms, 5), "algorithmic_bytes_per_launch": bytes_per_launch,
                    "achieved": round(bytes_per_launch / (ms * 1e-3) / 1e9, 2),
                    "frac": round(bytes_per_launch / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

        # the same operands copied (dst = peer, 2 bytes of traffic per byte written) two ways: by the library, one batch of
        # HcommLocalCopyOnThread calls = one k_copy_rows launch, and by the HIP runtime's own device-to-device copy, one
        # hipMemcpyAsync per segment - a yardstick that is not this library's code
        def lib_copy(k):
            h.check(h.HcommBatchModeStart(b"no_reuse_copy"), "HcommBatchModeStart")
            for d, p in bufs[k % sets]:
                h.check(h.HcommLocalCopyOnThread(thread, d.data_ptr(), p.data_ptr(), seg_bytes), "HcommLocalCopyOnThread")
            h.check(h.HcommBatchModeEnd(b"no_reuse_copy"), "HcommBatchModeEnd")

        def hip_copy(k):
            for d, p in bufs[k % sets]:
                rc = hip.hipMemcpyAsync(d.data_ptr(), p.data_ptr(), seg_bytes, 3, stream.cuda_stream)  # 3 = device to device
                if rc != 0:
                    raise RuntimeError("hipMemcpyAsync returned %d" % rc)

        row = timed(launch, 3 * nseg * seg_bytes, "k_reduce2_rows<bf16,SUM>")
        row.update({"segments": nseg, "segment_bytes": seg_bytes, "buffer_sets": sets})
        row["library_copy"] = timed(lib_copy, 2 * nseg * seg_bytes, "k_copy_rows")
        row["hip_memcpy_d2d"] = timed(hip_copy, 2 * nseg * seg_bytes, "hipMemcpyAsync, one call per segment")
        out[key] = row
        del bufs
    return out


def mesh_sweep(args, torch, h, dev, stream, thread, n, dt, unit):
    """Mesh one-shot allreduce SUM fp16, 8 ranks, 4 KiB .. 4 MiB per rank: latency (median of per-collective
    HIP-event times) and algorithmic GB/s (N(N+1)M bytes) for the fused single launch; the step-wise replay
    (N launches) is listed beside it."""
    points = []
    reps = max(args.steps, 100)
    # the floor: what one launch of this library costs in this harness when it moves next to nothing (a 16-byte copy
    # through HcommLocalCopyOnThread, one workgroup), timed the same two ways as the collectives below
    tiny = torch.zeros(64, dtype=torch.uint8, device=dev)
    for _ in range(10):
        h.HcommLocalCopyOnThread(thread, tiny.data_ptr() + 32, tiny.data_ptr(), 16)
    stream.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for a, b in ev:
        a.record(stream)
        h.HcommLocalCopyOnThread(thread, tiny.data_ptr() + 32, tiny.data_ptr(), 16)
        b.record(stream)
    stream.synchronize()
    ts = sorted(a.elapsed_time(b) * 1e3 for a, b in ev)
    floor_single = round(ts[len(ts) // 2], 2)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record(stream)
    for _ in range(reps):
        h.HcommLocalCopyOnThread(thread, tiny.data_ptr() + 32, tiny.data_ptr(), 16)
    b.record(stream)
    stream.synchronize()
    floor_pipelined = round(a.elapsed_time(b) * 1e3 / reps, 2)
    for m in [1 << s for s in range(12, 23)]:
        count = m // unit
        ins = make_inputs(torch, dev, n, count, "fp16")
        outs = [torch.zeros(m, dtype=torch.uint8, device=dev) for _ in range(n)]
        row = {"bytes_per_rank": m}
        for name, low in (("fused", h.Lowering.FUSED), ("stepwise", h.Lowering.STEPWISE)):
            plan = h.Plan(h.Alg.ALLREDUCE_MESH_ONESHOT, low, [t.data_ptr() for t in ins], [t.data_ptr() for t in outs],
                          count, dt, h.HcommReduceOp.SUM)
            for _ in range(10):
                plan.run(thread)
            stream.synchronize()
            ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
            for a, b in ev:
                a.record(stream)
                plan.run(thread)
                b.record(stream)
            stream.synchronize()
            ts = sorted(a.elapsed_time(b) * 1e3 for a, b in ev)
            row[name + "_us"] = round(ts[len(ts) // 2], 2)
            row[name + "_launches"] = plan.info.launches
            # back-to-back throughput: reps collectives between one pair of events
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            for _ in range(reps):
                plan.run(thread)
            b.record(stream)
            stream.synchronize()
            per = a.elapsed_time(b) * 1e3 / reps
            row[name + "_pipelined_us"] = round(per, 2)
            row[name + "_gbs"] = round(n * (n + 1) * m / (per * 1e-6) / 1e9, 1)
            plan.destroy()
        points.append(row)
    top = points[-1]
    return {"metric": "mesh one-shot allreduce SUM fp16, 8 simulated ranks: latency (us) and GB/s per message size",
            "value": top["fused_gbs"], "unit": "GB/s", "n_gpus": 1, "steps": reps, "warmup": 10,
            "ms_per_step": top["fused_pipelined_us"] / 1e3, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "fp16", "data": "synthetic",
            "config": {"workload": args.workload, "ranks": n, "algorithmic_bytes": "N(N+1)M = 72 M"},
            "launch_floor_us": {"single": floor_single, "pipelined": floor_pipelined,
                                "what": "a 16-byte HcommLocalCopyOnThread (one workgroup) in the same harness"},
            "sweep": points}


if __name__ == "__main__":
    main()
