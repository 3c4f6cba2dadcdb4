#!/usr/bin/env python3
"""Measures what the launch planner is audited against (run on the MI355X; writes planner_audit.json beside itself).

    python tests/golden/make_planner_audit.py [--quick] [--out PATH] [--instances 0,3 --update]

For every problem of a grid (int8 requant and fp16 GEMMs, A row-major, B column-major, LLM-like and square shapes
from 1 to 4096 rows; the ResNet-like conv layers of the benchmark) every instance that supports the problem is
timed with the workspace its own plan asks for: graph-replayed launches in 8 ms blocks until two blocks agree within
3 %, then the least of three more blocks (HIP events).
The file keeps microseconds per instance and the K runs the instance's plan used, so that the CPU test
tests/test_planner.py can hold the automatic choice (ckx_gemm_plan / ckx_conv2d_fwd_plan, pure host logic) against
the best measured instance without a GPU.
"""
import argparse
import json
import os
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

GEMM_NK = [(11008, 4096), (4096, 11008), (4096, 4096), (2048, 2048), (1024, 1024), (1024, 8192), (16384, 1024)]
GEMM_M = [1, 8, 16, 32, 48, 64, 128, 256, 512, 1024, 4096]
# (C, K, filter, HW, stride, pad) at N = 32 and 256: the benchmark's three layers, one more strided pointwise layer and
# the twenty distinct layers of the reference's whole-network run (script/profile_resnet50.sh:24-46)
CONV = [(64, 64, 3, 56, 1, 1), (256, 512, 1, 56, 2, 0), (512, 512, 3, 7, 1, 1), (128, 128, 3, 28, 1, 1),
        (256, 256, 3, 14, 1, 1), (64, 256, 1, 56, 1, 0), (1024, 2048, 1, 14, 2, 0),
        (1024, 256, 1, 14, 1, 0), (1024, 512, 1, 14, 1, 0), (128, 512, 1, 28, 1, 0), (128, 128, 3, 56, 2, 1),
        (2048, 512, 1, 7, 1, 0), (256, 1024, 1, 14, 1, 0), (256, 256, 3, 28, 2, 1), (256, 128, 1, 56, 1, 0),
        (512, 512, 3, 14, 2, 1), (512, 128, 1, 28, 1, 0), (512, 256, 1, 28, 1, 0), (512, 2048, 1, 7, 1, 0),
        (64, 64, 1, 56, 1, 0), (256, 64, 1, 56, 1, 0), (3, 64, 7, 224, 2, 3)]


def time_launch(launch, block_ms=8.0, max_settle_ms=400.0):
    """microseconds per launch: launches replayed from a HIP graph in blocks of about block_ms; blocks run until two in
    a row agree within 3 % (the clock governor has settled on this kernel: a light kernel is clocked down, and a
    cold one is clocked low), then the least of three more blocks counts."""
    import torch
    launch()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(20):
            launch()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def block(replays):
        e0.record()
        for _ in range(replays):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (20 * replays) * 1e3

    us = block(2)
    replays = max(2, int(block_ms * 1e3 / (20 * us)))
    t0, prev = time.perf_counter(), block(replays)
    while (time.perf_counter() - t0) * 1e3 < max_settle_ms:
        cur = block(replays)
        if abs(cur - prev) <= 0.03 * prev:
            break
        prev = cur
    return min(block(replays) for _ in range(3))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--quick", action="store_true", help="a fifth of the grid (smoke run of this script)")
    ap.add_argument("--only", default="i8,f16,conv",
                    help="comma-separated parts to measure: i8 (int8 GEMM rows), f16 (fp16 GEMM rows), conv; parts "
                         "measured in separate runs are merged by hand (same keys)")
    ap.add_argument("--out", default=None, help="where to write the table (default: planner_audit.json beside this script)")
    ap.add_argument("--instances", default=None,
                    help="comma-separated GEMM instance indices: time only these columns (with --update, after a kernel "
                         "behind an instance has changed)")
    ap.add_argument("--update", action="store_true",
                    help="start from the table beside this script: rows are matched by their problem, the measured columns "
                         "and the automatic choice replace the old entries, everything else is kept")
    args = ap.parse_args()
    import torch
    import composable_kernel_amd as ck
    from composable_kernel_amd import capi
    L = capi.lib()
    stream = lambda: torch.cuda.current_stream().cuda_stream
    out = {"device": torch.cuda.get_device_name(0), "library": L.ckx_version().decode(),
           "auto": "the automatic choice [instance, K runs] of the library that was measured, with 256 MiB of workspace on offer",
           "protocol": "per instance: graph-replayed launches in 8 ms blocks until two agree within 3 %, then the least of three more blocks, HIP events, microseconds",
           "gemm": [], "conv": []}
    n_inst = L.ckx_num_instances(capi.OP_GEMM_I8)
    columns = None if args.instances is None else {int(x) for x in args.instances.split(",")}
    old = None
    if args.update:
        with open(os.path.join(HERE, "planner_audit.json")) as f:
            old = json.load(f)
        out["conv"] = old["conv"]
        out["updated"] = "columns " + (args.instances or "all") + " of the GEMM rows re-measured with this library"
    ws = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
    only = set(args.only.split(","))
    if not args.update and not only & {"i8", "f16"} and os.path.exists(os.path.join(HERE, "planner_audit.json")):
        with open(os.path.join(HERE, "planner_audit.json")) as f:   # a conv-only run keeps the GEMM rows it finds
            out["gemm"] = json.load(f)["gemm"]
    grid = [(kind, M, N, K) for kind in ("i8", "f16") if kind in only for (N, K) in GEMM_NK for M in GEMM_M]
    if args.quick:
        grid = grid[::5]
    for kind, M, N, K in grid:
        tdt = torch.int8 if kind == "i8" else torch.float16
        mk = (lambda s: torch.randint(-8, 9, s, dtype=torch.int8, device="cuda")) if kind == "i8" else \
             (lambda s: (torch.rand(s, device="cuda") * 2 - 1).to(torch.float16))
        a, b, c = mk((M, K)), mk((N, K)), torch.empty((M, N), dtype=tdt, device="cuda")
        cls = ck.DeviceGemmInt8 if kind == "i8" else ck.DeviceGemmF16
        c_op = ck.RequantReluRequant(0.02, 0.4, rounded=True) if kind == "i8" else None
        opf = capi.OP_GEMM_I8 if kind == "i8" else capi.OP_GEMM_F16
        epi = capi.EPI_REQUANT_RND if kind == "i8" else capi.EPI_PASSTHROUGH
        row = {"op": kind, "M": M, "N": N, "K": K, "us": {}, "k_runs": {}}
        if old is not None:
            prev = [r for r in old["gemm"] if (r["op"], r["M"], r["N"], r["K"]) == (kind, M, N, K)]
            if prev:
                row["us"], row["k_runs"] = dict(prev[0]["us"]), dict(prev[0]["k_runs"])
        for inst in range(n_inst - 1):        # (the element-wise instance is never the choice for an aligned problem)
            if columns is not None and inst not in columns:
                continue
            op = cls(inst)
            arg = op.MakeArgumentPointer(a, b, c, M, N, K, K, K, N, None, None, c_op)
            if not op.IsSupportedArgument(arg):
                continue
            need = op.GetWorkSpaceSize(arg)
            if need > ws.numel():
                continue
            op.SetWorkSpacePointer(arg, ws, need)
            _, runs = capi.gemm_plan(opf, M, N, K, epilogue=epi, workspace_bytes=need, instance=inst)

            def launch(op=op, arg=arg):
                st = op._launch(arg, stream())
                assert st == 0, capi.last_error()
            row["us"][str(inst)] = round(time_launch(launch), 2)
            row["k_runs"][str(inst)] = runs
        row["auto"] = list(capi.gemm_plan(opf, M, N, K, epilogue=epi, workspace_bytes=ws.numel()))
        out["gemm"].append(row)
        print(row, flush=True)
    if old is not None:   # rows outside this run's grid are kept as they were, in the table's order
        done = {(r["op"], r["M"], r["N"], r["K"]): r for r in out["gemm"]}
        out["gemm"] = [done.get((r["op"], r["M"], r["N"], r["K"]), r) for r in old["gemm"]]
    n_conv = L.ckx_num_instances(capi.OP_CONV2D_FWD_I8)
    cgrid = [(kind, n, *layer) for kind in ("i8", "f16") for n in (32, 256) for layer in CONV] \
        if "conv" in only and not args.update else []
    if args.quick:
        cgrid = cgrid[::5]
    for kind, Nb, C_, K, f, HW, st_, pd in cgrid:
        Ho = (HW + 2 * pd - f) // st_ + 1
        tdt = torch.int8 if kind == "i8" else torch.float16
        mk = (lambda s: torch.randint(-5, 6, s, dtype=torch.int8, device="cuda")) if kind == "i8" else \
             (lambda s: (torch.rand(s, device="cuda") * 2 - 1).to(torch.float16))
        x, w, y = mk((Nb, HW, HW, C_)), mk((K, f, f, C_)), torch.empty((Nb, Ho, Ho, K), dtype=tdt, device="cuda")
        cls = ck.DeviceConv2dFwdInt8 if kind == "i8" else ck.DeviceConv2dFwdF16
        c_op = ck.RequantReluRequant(0.01, 0.5, rounded=True) if kind == "i8" else None
        opf = capi.OP_CONV2D_FWD_I8 if kind == "i8" else capi.OP_CONV2D_FWD_F16
        epi = capi.EPI_REQUANT_RND if kind == "i8" else capi.EPI_PASSTHROUGH
        desc = capi.Conv2dDesc(Nb, K, C_, HW, HW, f, f, Ho, Ho, st_, st_, 1, 1, pd, pd, pd, pd)
        row = {"op": kind, "N": Nb, "C": C_, "K": K, "filter": f, "HW": HW, "stride": st_, "pad": pd, "us": {}, "k_runs": {}}
        for inst in range(n_conv - 1):
            op = cls(inst)
            arg = op.MakeArgumentPointer(x, w, y, Nb, K, C_, [HW, HW], [f, f], [Ho, Ho], [st_, st_], [1, 1], [pd, pd], [pd, pd],
                                         None, None, c_op)
            if not op.IsSupportedArgument(arg):
                continue
            need = op.GetWorkSpaceSize(arg)
            if need > ws.numel():
                continue
            op.SetWorkSpacePointer(arg, ws, need)
            _, runs = capi.conv2d_fwd_plan(opf, desc, epi, need, inst)

            def launch(op=op, arg=arg):
                st = op._launch(arg, stream())
                assert st == 0, capi.last_error()
            row["us"][str(inst)] = round(time_launch(launch), 2)
            row["k_runs"][str(inst)] = runs
        row["auto"] = list(capi.conv2d_fwd_plan(opf, desc, epi, ws.numel()))
        out["conv"].append(row)
        print(row, flush=True)
    path = args.out or os.path.join(HERE, "planner_audit.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=0, separators=(",", ":"))
    print("wrote", path)


if __name__ == "__main__":
    main()
