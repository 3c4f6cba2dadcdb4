#!/usr/bin/env python3
"""Benchmark of the MFMA GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--all] [--no-cpu]

A "step" is one launch of the workload's kernel over synthetic inputs that are already resident
in HBM. The default workload is the fp16 GEMM at 4096^3 on which the
metric (TFLOP/s and fraction of the dense fp16 MFMA peak) is quoted; the int8 half of the metric
(4096^3 requant GEMM, TOP/s) and every other config are measured too and attached under "also".
Prints ONE JSON line on stdout.

Timing: a clock-settling phase, W untimed launches, then exactly K launches between two events
recorded on the launch stream (torch's current stream, whose handle is what the C ABI receives),
bracketed by device synchronisation; wall-clock over the same region gives ms_per_step. The K
launches are replayed from a HIP graph captured from the same C-ABI calls, so that the GPU runs
them back to back even for kernels shorter than a Python call (--no-graph launches eagerly).

Clock settling: a GPU that was idle runs its first launches several hundred MHz below its
operating point and takes tens of milliseconds of load to leave that state, so a short run
(--steps 20 --warmup 5) would time the ramp, not the kernel. Before the W warm-up launches the
same kernel is therefore replayed, untimed, in blocks until the mean launch time of a block stops
changing (and at least --settle-ms of load have passed); the line discloses it ("settle_launches",
"settle_ms") and also carries the figure WITHOUT it under "from_idle": 1 warm-up + 10 timed
launches from the idle GPU, the reference's own timing protocol
(include/ck/device_utility/kernel_launch.hpp:20-62).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"f16": 2516.6, "bf16": 2516.6, "i8": 5033.2}   # dense MFMA TFLOP/s / TOP/s, 256 CUs x 2.4 GHz
HBM_PEAK_GBS = 8000.0
PEAK_CLOCK_MHZ = 2400.0   # the engine clock the published MFMA peaks are quoted at
# Bytes crossing the L2 <-> fabric boundary per launch, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# scaled by a 256 MiB copy in the same run (profiles/gemm_w4_fp16_int8_4096_hbm_traffic.md).
MEASURED_TRAFFIC = {"fp16_gemm_4096": 2.350e8, "int8_requant_gemm_4096": 1.180e8}
TRAFFIC_SOURCE = ("cited, not measured in this run: profiles/gemm_w4_fp16_int8_4096_hbm_traffic.md "
                  "(rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, each scaled by a 256 MiB copy in the same run)")


def _conv_workload(name, dtype, C, K, f, HW, st, pd, N=256, fused=None):
    """fused: None, "bias_relu" or "bias_relu_add" (fp16: + bias[K], ReLU, + residual NHWK)."""
    Ho = (HW + 2 * pd - f) // st + 1
    ops = 2.0 * N * K * Ho * Ho * C * f * f
    es = 1 if dtype == "i8" else 2
    touched_in = N * HW * HW * C if st == 1 or f > 1 else N * Ho * Ho * C
    out = N * Ho * Ho * K
    byts = (touched_in + K * f * f * C + out + (K if fused else 0) + (out if fused == "bias_relu_add" else 0)) * es
    return dict(name=name, kind="conv", dtype=dtype, N=N, C=C, K=K, f=f, HW=HW, st=st, pd=pd, ops=ops, bytes=byts,
                fused=fused)


def _conv3d_workload(name, dtype, C, K, f, DHW, st, pd, N, dil=1):
    """Three spatial dimensions, NDHWC / KZYXC / NDHWK, cubic extents."""
    Do = (DHW + 2 * pd - ((f - 1) * dil + 1)) // st + 1
    es = 1 if dtype == "i8" else 2
    ops = 2.0 * N * K * Do ** 3 * C * f ** 3
    byts = (N * DHW ** 3 * C + K * f ** 3 * C + N * Do ** 3 * K) * es
    return dict(name=name, kind="conv", ndim=3, dtype=dtype, N=N, C=C, K=K, f=f, HW=DHW, st=st, pd=pd, dil=dil, ops=ops,
                bytes=byts, fused=None)


def _gemm_workload(name, dtype, M, N, K, values=5, scales=(0.5, 0.03), fused=None, batch=1, layout="mk_nk", init="uniform"):
    """fused: None, "bias_relu" (fp16: E = AddRelu(half(A*B), bias row)), "bilinear" (E = alpha * A*B + beta * D, D a
    full [M,N] tensor, example 02) or "add_add_fastgelu" (E = fast_gelu(A*B + bias row + D1), example 04);
    batch > 1: strided batched GEMM;
    layout: how A ("mk" row-major / "km" column-major) and B ("nk" column-major / "kn" row-major) are stored."""
    es = 1 if dtype == "i8" else 2
    d_elems = {None: 0, "bias_relu": N, "bilinear": M * N, "add_add_fastgelu": N + M * N}[fused]
    return dict(name=name, kind="gemm", dtype=dtype, M=M, N=N, K=K, values=values, scales=scales, batch=batch,
                layout=layout, init=init,
                ops=2.0 * M * N * K * batch, bytes=(M * K + N * K + M * N + d_elems) * es * batch,
                fused=fused)


WORKLOADS = {}
for w in (
    [_gemm_workload("fp16_gemm_4096", "f16", 4096, 4096, 4096),
     _gemm_workload("int8_requant_gemm_4096", "i8", 4096, 4096, 4096),
     _gemm_workload("int8_requant_gemm_1024", "i8", 1024, 1024, 1024)]
    + [_gemm_workload(f"int8_requant_llm_m{m}_n11008_k4096", "i8", m, 11008, 4096, 8, (0.02, 0.4)) for m in (1, 16, 128, 4096)]
    + [_gemm_workload(f"int8_requant_llm_m{m}_n4096_k11008", "i8", m, 4096, 11008, 8, (0.02, 0.4)) for m in (1, 16, 128, 4096)]
    + [_conv_workload(f"conv_{dt}_c64_k64_3x3_56", dt, 64, 64, 3, 56, 1, 1) for dt in ("f16", "i8")]
    + [_conv_workload(f"conv_{dt}_c256_k512_1x1_56_s2", dt, 256, 512, 1, 56, 2, 0) for dt in ("f16", "i8")]
    + [_conv_workload(f"conv_{dt}_c512_k512_3x3_7", dt, 512, 512, 3, 7, 1, 1) for dt in ("f16", "i8")]
    + [_gemm_workload("fp16_batched_gemm_g16_1024", "f16", 1024, 1024, 1024, batch=16),
       _gemm_workload("bf16_gemm_4096", "bf16", 4096, 4096, 4096)]
    + [_gemm_workload(f"fp16_gemm_4096_{lay}", "f16", 4096, 4096, 4096, layout=lay) for lay in ("km_kn", "km_nk", "mk_kn")]
    + [_gemm_workload(f"int8_requant_gemm_4096_{lay}", "i8", 4096, 4096, 4096, layout=lay) for lay in ("km_kn", "km_nk", "mk_kn")]
    + [_gemm_workload("fp16_gemm_bias_relu_4096", "f16", 4096, 4096, 4096, fused="bias_relu"),
       _gemm_workload("fp16_gemm_bilinear_4096", "f16", 4096, 4096, 4096, fused="bilinear"),
       _gemm_workload("fp16_gemm_add_add_fastgelu_4096", "f16", 4096, 4096, 4096, fused="add_add_fastgelu"),
       _gemm_workload("fp16_gemm_4096_integer_init", "f16", 4096, 4096, 4096, init="integer"),
       _conv_workload("conv_f16_c64_k64_3x3_56_bias_relu_add", "f16", 64, 64, 3, 56, 1, 1, fused="bias_relu_add"),
       _conv_workload("conv_f16_c256_k512_1x1_56_s2_bias_relu", "f16", 256, 512, 1, 56, 2, 0, fused="bias_relu")]
    # three spatial dimensions: the reference's device-test default (conv3d_fwd.cpp:76-77) and a larger 3x3x3 layer
    + [_conv3d_workload("conv3d_f16_n4_c64_k256_3x3x3_28_s2_d2", "f16", 64, 256, 3, 28, 2, 2, 4, dil=2),
       _conv3d_workload("conv3d_f16_n16_c64_k64_3x3x3_32", "f16", 64, 64, 3, 32, 1, 1, 16),
       _conv3d_workload("conv3d_i8_n16_c64_k64_3x3x3_32", "i8", 64, 64, 3, 32, 1, 1, 16)]
    + [dict(name="gemm_gemm_f16_b64_512x64x512x64", kind="gemm_gemm", dtype="f16", G=64, M=512, N=512, K=64, O=64,
            ops=2.0 * 64 * 512 * 512 * 64 * 2, bytes=4 * 64 * 512 * 64 * 2),
       # the same shapes with a softmax between the GEMMs (attention): 64 heads of 512 x 512 scores, and a long one
       dict(name="gemm_softmax_gemm_f16_b64_512x64x512x64", kind="gemm_gemm", softmax=True, dtype="f16", G=64, M=512,
            N=512, K=64, O=64, ops=2.0 * 64 * 512 * 512 * 64 * 2, bytes=4 * 64 * 512 * 64 * 2),
       dict(name="gemm_softmax_gemm_f16_b64_4096x64x4096x64", kind="gemm_gemm", softmax=True, dtype="f16", G=64, M=4096,
            N=4096, K=64, O=64, ops=2.0 * 64 * 4096 * 4096 * 64 * 2, bytes=4 * 64 * 4096 * 64 * 2)]
):
    WORKLOADS[w["name"]] = w

# The layers the reference's own whole-network script drives through ckProfiler at N = 256
# (script/profile_resnet50.sh:24-46: the de-duplicated list, run as `conv_fwd`): (K, C, filter, H = W, stride, pad)
RESNET50_LAYERS = [
    (256, 1024, 1, 14, 1, 0), (512, 1024, 1, 14, 1, 0), (128, 128, 3, 28, 1, 1), (512, 128, 1, 28, 1, 0),
    (128, 128, 3, 56, 2, 1), (512, 2048, 1, 7, 1, 0), (1024, 256, 1, 14, 1, 0), (256, 256, 3, 14, 1, 1),
    (256, 256, 3, 28, 2, 1), (128, 256, 1, 56, 1, 0), (64, 256, 1, 56, 1, 0), (512, 512, 3, 14, 2, 1),
    (128, 512, 1, 28, 1, 0), (256, 512, 1, 28, 1, 0), (2048, 512, 1, 7, 1, 0), (512, 512, 3, 7, 1, 1),
    (256, 64, 1, 56, 1, 0), (64, 64, 1, 56, 1, 0), (64, 64, 3, 56, 1, 1), (64, 3, 7, 224, 2, 3)]
# ... and the distinct (operation, layer) pairs of its fused run (:47-99): conv_fwd_bias_relu_add on these layers, on
# top of conv_fwd_bias_relu on every layer above
RESNET50_BIAS_RELU_ADD = [(256, 64, 1, 56, 1, 0), (512, 128, 1, 28, 1, 0), (1024, 256, 1, 14, 1, 0), (2048, 512, 1, 7, 1, 0)]


def resnet50_workloads(N=256):
    out = []
    for (K, C, f, HW, st, pd) in RESNET50_LAYERS:
        tag = f"c{C}_k{K}_{f}x{f}_{HW}" + (f"_s{st}" if st > 1 else "")
        for dt in ("f16", "i8"):
            out.append(_conv_workload(f"conv_{dt}_{tag}", dt, C, K, f, HW, st, pd, N))
        out.append(_conv_workload(f"conv_f16_{tag}_bias_relu", "f16", C, K, f, HW, st, pd, N, fused="bias_relu"))
        if (K, C, f, HW, st, pd) in RESNET50_BIAS_RELU_ADD:
            out.append(_conv_workload(f"conv_f16_{tag}_bias_relu_add", "f16", C, K, f, HW, st, pd, N, fused="bias_relu_add"))
    return out


def make_launcher(w, instance=-1, rotate=1):
    """Allocates the workload's synthetic operands on the GPU, returns the launch function.
    rotate > 1 (GEMM workloads): that many distinct copies of the B matrix, used round-robin, so
    that a weight matrix smaller than the 256 MB Infinity Cache is read from HBM every time."""
    import torch
    import composable_kernel_amd as ck
    from composable_kernel_amd import capi
    from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8

    keep = []

    def dev(a):
        t = torch.from_numpy(a).cuda()
        keep.append(t)
        return t

    if w["kind"] == "gemm":
        M, N, K = w["M"], w["N"], w["K"]
        la, lb = w.get("layout", "mk_nk").split("_")
        a_shape, b_shape = ((M, K) if la == "mk" else (K, M)), ((N, K) if lb == "nk" else (K, N))
        lay = dict(ALayout=ck.RowMajor if la == "mk" else ck.ColumnMajor, BLayout=ck.ColumnMajor if lb == "nk" else ck.RowMajor)
        sa, sb = a_shape[1], b_shape[1]
        if w["dtype"] == "i8":
            a, b = dev(uniform_int8(a_shape, -w["values"], w["values"], 1)), dev(uniform_int8(b_shape, -w["values"], w["values"], 2))
            c = torch.empty((M, N), dtype=torch.int8, device="cuda")
            op = ck.DeviceGemmInt8(instance, **lay)
            cop = ck.RequantReluRequant(w["scales"][0], w["scales"][1], rounded=True)
        else:
            if w.get("init") == "integer":
                # the reference profiler's initialisation 1 (its published runs): integers in [-5, 5]
                a = dev(uniform_int8(a_shape, -5, 5, 1).astype(np.float16))
                b = dev(uniform_int8(b_shape, -5, 5, 2).astype(np.float16))
            elif w.get("init") == "zeros":
                # no operand bit toggles: the kernel at the full engine clock (the power limit does not bind)
                a, b = dev(np.zeros(a_shape, np.float16)), dev(np.zeros(b_shape, np.float16))
            else:
                a, b = dev(uniform_f16(a_shape, -1, 1, 1)), dev(uniform_f16(b_shape, -1, 1, 2))
            c = torch.empty((M, N), dtype=torch.float16, device="cuda")
            op = ck.DeviceGemmF16(instance, **lay)
            cop = ck.PassThrough()
        G = w.get("batch", 1)
        if w["dtype"] == "bf16":
            from composable_kernel_amd.host_tensor import uniform_bf16
            a = dev(uniform_bf16((M, K), -1, 1, 1).view(np.int16))
            b = dev(uniform_bf16((N, K), -1, 1, 2).view(np.int16))
            c = torch.empty((M, N), dtype=torch.int16, device="cuda")
            op = ck.DeviceGemmBF16(instance)
            make = lambda bb: op.MakeArgumentPointer(a, bb, c, M, N, K, K, K, N)
        elif G > 1:
            a, b = dev(uniform_f16((G * M, K), -1, 1, 1)), dev(uniform_f16((G * N, K), -1, 1, 2))
            c = torch.empty((G * M, N), dtype=torch.float16, device="cuda")
            op = ck.DeviceBatchedGemmF16(instance)
            make = lambda bb: op.MakeArgumentPointer(a, bb, c, M, N, K, K, K, N, M * K, N * K, M * N, G)
        elif w.get("fused") == "bias_relu":
            bias = dev(uniform_f16((N,), -1, 1, 9))
            op = ck.DeviceGemmMultipleDF16(instance)
            make = lambda bb: op.MakeArgumentPointer(a, bb, [bias], c, M, N, K, K, K, [0], N, None, None, ck.AddRelu())
        elif w.get("fused") in ("bilinear", "add_add_fastgelu"):
            bias, full = dev(uniform_f16((N,), -1, 1, 9)), dev(uniform_f16((M, N), -1, 1, 10))
            op = ck.DeviceGemmMultipleDF16(instance)
            if w["fused"] == "bilinear":
                make = lambda bb: op.MakeArgumentPointer(a, bb, [full], c, M, N, K, K, K, [N], N, None, None,
                                                         ck.Bilinear(0.5, 1.5))
            else:
                make = lambda bb: op.MakeArgumentPointer(a, bb, [bias, full], c, M, N, K, K, K, [0, N], N, None, None,
                                                         ck.AddAddFastGelu())
        else:
            make = lambda bb: op.MakeArgumentPointer(a, bb, c, M, N, K, sa, sb, N, None, None, cop)
        arg = make(b)
        more_args = []
        for _ in range(rotate - 1):
            b2 = b.clone()
            keep.append(b2)
            more_args.append(make(b2))
    elif w["kind"] == "conv":
        N, C, K, f, HW, st, pd = (w[k] for k in ("N", "C", "K", "f", "HW", "st", "pd"))
        nd, dil = w.get("ndim", 2), w.get("dil", 1)
        Ho = (HW + 2 * pd - ((f - 1) * dil + 1)) // st + 1
        if w["dtype"] == "i8":
            i, wt = dev(uniform_int8((N, *[HW] * nd, C), -5, 5, 3)), dev(uniform_int8((K, *[f] * nd, C), -5, 5, 4))
            c = torch.empty((N, *[Ho] * nd, K), dtype=torch.int8, device="cuda")
            op = ck.DeviceConv2dFwdInt8(instance) if nd == 2 else ck.DeviceConvNdFwdInt8(nd, instance)
            cop = ck.RequantReluRequant(0.01, 0.5, rounded=True)
        else:
            i, wt = dev(uniform_f16((N, *[HW] * nd, C), -1, 1, 3)), dev(uniform_f16((K, *[f] * nd, C), -1, 1, 4))
            c = torch.empty((N, *[Ho] * nd, K), dtype=torch.float16, device="cuda")
            op = ck.DeviceConv2dFwdF16(instance) if nd == 2 else ck.DeviceConvNdFwdF16(nd, instance)
            cop = ck.PassThrough()
        geom = (N, K, C, [HW] * nd, [f] * nd, [Ho] * nd, [st] * nd, [dil] * nd, [pd] * nd, [pd] * nd, None, None)
        if w.get("fused"):
            op = ck.DeviceConv2dFwdBiasActivationF16(instance)
            bias = dev(uniform_f16((K,), -1, 1, 7))
            if w["fused"] == "bias_relu_add":
                resi = dev(uniform_f16((N, Ho, Ho, K), -1, 1, 8))
                arg = op.MakeArgumentPointer(i, wt, c, bias, resi, *geom, ck.AddReluAdd())
            else:
                arg = op.MakeArgumentPointer(i, wt, c, bias, *geom, ck.AddRelu())
        else:
            arg = op.MakeArgumentPointer(i, wt, c, *geom, cop)
    else:
        G, M, N, K, O = (w[k] for k in ("G", "M", "N", "K", "O"))
        a, b0, b1 = (dev(uniform_f16(s, -0.5, 0.5, 5 + j)) for j, s in enumerate([(G, M, K), (G, N, K), (G, N, O)]))
        c = torch.empty((G, M, O), dtype=torch.float16, device="cuda")
        if w.get("softmax"):
            op = ck.DeviceBatchedGemmSoftmaxGemmF16(instance)
            arg = op.MakeArgumentPointer(a, b0, b1, c, M, N, K, O, G, K, K, O, O, M * K, N * K, N * O, M * O,
                                         None, None, ck.Scale(K ** -0.5))
        else:
            op = ck.DeviceBatchedGemmGemmF16(instance)
            arg = op.MakeArgumentPointer(a, b0, b1, c, M, N, K, O, G, K, K, O, O, M * K, N * K, N * O, M * O)
    keep.append(c)
    if not op.IsSupportedArgument(arg):
        raise RuntimeError(f"{w['name']}: not supported: {capi.last_error()}")
    need = op.GetWorkSpaceSize(arg)
    if need:   # optional split-K scratch, allocated once outside the timed region
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        keep.append(ws)
        op.SetWorkSpacePointer(arg, ws)
    args = [arg]
    if w["kind"] == "gemm":
        for extra in more_args:
            if need:
                op.SetWorkSpacePointer(extra, ws)
            args.append(extra)
    turn = [0]

    def launch():
        st_ = op._launch(args[turn[0] % len(args)], torch.cuda.current_stream().cuda_stream)
        turn[0] += 1
        if st_ != 0:
            raise RuntimeError(capi.last_error())

    launch.keep = keep
    return launch


def _figures(w, ev_ms):
    tput = w["ops"] / (ev_ms * 1e-3) / 1e12
    gbs = w["bytes"] / (ev_ms * 1e-3) / 1e9
    compute_frac = tput / PEAK[w["dtype"]]
    hbm_frac = gbs / HBM_PEAK_GBS
    return dict(tput=tput, gbs=gbs, mfma_frac=compute_frac, hbm_frac=hbm_frac,
                bound="mfma" if compute_frac >= hbm_frac else "hbm")


def _sclk_under_load(chunk, chunk_ms, busy_ms=1500.0):
    """Engine clock (MHz) read with rocm-smi while the same launches keep replaying, after the timed region: about
    busy_ms of work is queued, the clock is read up to three times, and a reading counts only if the queue was
    still busy after it. Empty when rocm-smi is missing, slow or prints something else."""
    import re
    import subprocess
    import torch
    done = torch.cuda.Event()
    for _ in range(max(1, int(busy_ms / max(chunk_ms, 1e-3)))):
        chunk()
    done.record()
    seen = []
    try:
        for _ in range(3):
            txt = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=5).stdout
            m = re.search(r"sclk clock level[^\n]*\((\d+)Mhz\)", txt)
            if done.query():
                break
            if m:
                seen.append(int(m.group(1)))
    except (OSError, subprocess.SubprocessError):
        pass
    torch.cuda.synchronize()
    return seen


def vendor_launcher(w):
    """The vendor library's kernel for the same problem on operands of the same distribution, for the figure
    beside the headline rows: torch.matmul (hipBLASLt) for fp16, torch._int_mm for int8 (int32 output: it does
    not requantize, so it writes four times the C bytes of the int8 row)."""
    import torch
    from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8
    M, N, K = w["M"], w["N"], w["K"]
    if w["dtype"] == "f16":
        a = torch.from_numpy(uniform_f16((M, K), -1, 1, 1)).cuda()
        bt = torch.from_numpy(uniform_f16((N, K), -1, 1, 2)).cuda().t()
        c = torch.empty((M, N), dtype=torch.float16, device="cuda")
        fn = lambda: torch.matmul(a, bt, out=c)
    else:
        a = torch.from_numpy(uniform_int8((M, K), -5, 5, 1)).cuda()
        bt = torch.from_numpy(uniform_int8((N, K), -5, 5, 2)).cuda().t()
        c = torch.empty((M, N), dtype=torch.int32, device="cuda")
        fn = lambda: torch._int_mm(a, bt, out=c)
    fn.keep = [a, bt, c]
    return fn


def time_workload(w, steps, warmup, instance=-1, use_graph=True, rotate=1, settle_ms=300.0, from_idle=False,
                  sample_clock=False, launch=None):
    """[from_idle: 1 + 10 eager launches first], clock settling, W untimed launches, then exactly K timed
    ones. The K launches are replayed from a HIP graph (captured once from the same C-ABI calls) so that
    kernels run back to back on the GPU even when one kernel is shorter than a Python call;
    use_graph=False launches eagerly."""
    import torch
    launch = launch or make_launcher(w, instance, rotate)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    idle = None
    if from_idle:
        # the reference's protocol (kernel_launch.hpp:20-62): one warm-up launch, a device
        # synchronisation, ten launches between two events, the mean
        launch()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(10):
            launch()
        e1.record()
        torch.cuda.synchronize()
        idle = e0.elapsed_time(e1) / 10
    # launches per captured graph: a divisor of K that walks the rotation a whole number of times
    cands = [d for d in range(1, min(steps, 50) + 1) if steps % d == 0 and d % rotate == 0]
    per_graph = max(cands) if cands else rotate
    graph = None
    if use_graph:
        launch()   # (the library's one-time function attributes are set outside the capture)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(per_graph):
                launch()

    def chunk():
        if graph is not None:
            graph.replay()
        else:
            for _ in range(per_graph):
                launch()

    # ---- clock settling: blocks of launches until a block's mean time stops moving ----------
    settle_launches, settle_total, blocks = 0, 0.0, []
    if settle_ms > 0:
        est = None
        while settle_total < 4000.0:
            n_chunks = 4 if est is None else max(4, min(400, int(25.0 / max(est * per_graph, 1e-3))))  # ~25 ms blocks
            e0.record()
            for _ in range(n_chunks):
                chunk()
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            est = ms / (n_chunks * per_graph)
            settle_launches += n_chunks * per_graph
            settle_total += ms
            blocks.append(est)
            if settle_total >= settle_ms and len(blocks) >= 3 and abs(blocks[-1] - blocks[-2]) <= 0.01 * blocks[-2] \
                    and abs(blocks[-1] - blocks[-3]) <= 0.015 * blocks[-3]:
                break
    for _ in range(warmup):
        launch()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    if graph is not None:
        for _ in range(steps // per_graph):
            graph.replay()
    else:
        for _ in range(steps):
            launch()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms = e0.elapsed_time(e1) / steps
    out = dict(workload=w["name"], dtype=w["dtype"], ms=ev_ms, wall_ms=wall_ms, settle_launches=settle_launches,
               settle_ms=settle_total, settle_blocks_us=[round(b * 1e3, 1) for b in blocks], **_figures(w, ev_ms))
    if sample_clock:
        out["sclk_mhz"] = _sclk_under_load(chunk, ev_ms * per_graph)
    if idle is not None:
        out["from_idle_ms"] = idle
    return out


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_threads():
    """Threads of the CPU leg: the cores this process may run on -- its affinity mask, and where the host
    is shared (a GPU box grants each GPU's job a share of the cores and says so in OMP_NUM_THREADS) that share.
    The reference's host operators use std::thread::hardware_concurrency() threads (reference_gemm.hpp:83-85,
    host_tensor.hpp:174-193), which is the same number on a host that is one's own."""
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    share = os.environ.get("OMP_NUM_THREADS", "")
    if share.isdigit() and int(share) > 0:
        n = min(n, int(share))
    return max(1, n)


def cpu_baseline(w, threads=None, budget_seconds=30.0):
    """The oracle's literal ReferenceGemm restatement on the host cores of this box: the WHOLE problem when a
    probe says it fits the time budget, else a bounded row sample of it (stated in "sample")."""
    from oracle import lit
    from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8
    threads = threads or cpu_threads()
    N, K = w["N"], w["K"]
    if w["dtype"] == "f16":
        b = uniform_f16((N, K), -1, 1, 2)
        mk = lambda m: uniform_f16((m, K), -1, 1, 1)
        run = lambda a: lit.gemm_f16(a, b.T, nthreads=threads)
    else:
        b = uniform_int8((N, K), -5, 5, 2)
        mk = lambda m: uniform_int8((m, K), -5, 5, 1)
        run = lambda a: lit.gemm_i8(a, b.T, lit.EPI_REQUANT_RND, 0.5, 0.03, nthreads=threads)
    m0 = min(w["M"], 2 * threads)
    t0 = time.perf_counter()
    run(mk(m0))
    dt = max(time.perf_counter() - t0, 1e-4)
    rows = int(min(w["M"], max(m0, m0 * budget_seconds / dt)))
    a = mk(rows)
    t0 = time.perf_counter()
    run(a)
    dt = time.perf_counter() - t0
    unit = "TFLOP/s" if w["dtype"] == "f16" else "TOP/s"
    what = "the whole" if rows == w["M"] else f"{rows} of {w['M']} rows of the same"
    port = {"value": 2.0 * rows * N * K / dt / 1e12, "unit": unit, "cores": threads, "kind": "port",
            "host_cores": os.cpu_count(), "cpu_model": _cpu_model(),
            "sample": f"{what} {w['M']}x{N}x{K} problem, literal ReferenceGemm restatement "
                      f"(oracle/ck_oracle.cpp), {threads} threads, {dt:.1f} s"}
    # The reference's OWN host operator (ReferenceGemm compiled in place from the reference tree into oracle/_ref,
    # where that build exists): slower than the restatement (tensor accessors through descriptors), so a row sample
    # sized for about ten seconds. It starts std::thread::hardware_concurrency() threads whatever the job may use.
    import oracle
    ref = oracle.load_ref()
    if ref is None:
        return port
    ref_run = (lambda a: ref.gemm_f16(a, b.T)) if w["dtype"] == "f16" else \
              (lambda a: ref.gemm_i8_requant(a, b.T, lit.EPI_REQUANT_RND, 0.5, 0.03))
    m0 = min(w["M"], 64)
    t0 = time.perf_counter()
    ref_run(mk(m0))
    dt0 = max(time.perf_counter() - t0, 1e-4)
    rrows = int(min(w["M"], max(m0, m0 * 10.0 / dt0)))
    a = mk(rrows)
    t0 = time.perf_counter()
    ref_run(a)
    rdt = time.perf_counter() - t0
    what = "the whole" if rrows == w["M"] else f"{rrows} of {w['M']} rows of the same"
    return {"value": 2.0 * rrows * N * K / rdt / 1e12, "unit": unit, "cores": min(threads, os.cpu_count() or threads),
            "kind": "reference", "reference_threads": os.cpu_count(), "host_cores": os.cpu_count(),
            "cpu_model": _cpu_model(),
            "sample": f"{what} {w['M']}x{N}x{K} problem, the reference's ReferenceGemm host operator compiled in place "
                      f"(oracle/_ref), {rdt:.1f} s; it starts one thread per host CPU, this job may use {threads}",
            "port": port}


def cpu_baseline_row(w, seconds=2.0, threads=None):
    """The reference's own host operator for this workload's family (compiled in place into oracle/_ref: ReferenceGemm,
    ReferenceConvFwd, ReferenceBatchedGemm; the oracle's restatement where that build is absent), timed on a sample of
    the same problem -- rows of A, images, or batches -- sized by a probe for about `seconds` of work."""
    import oracle
    from oracle import lit
    from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8
    threads = threads or cpu_threads()
    ref = oracle.load_ref()
    kind = "reference" if ref is not None else "port"
    dt = w["dtype"]
    if w["kind"] == "gemm":
        M, N, K, G = w["M"], w["N"], w["K"], w.get("batch", 1)
        unit_name, total, per_unit = "rows", M * G, 2.0 * N * K
        if dt == "i8":
            b = uniform_int8((N, K), -w["values"], w["values"], 2)
            mk = lambda m: uniform_int8((m, K), -w["values"], w["values"], 1)
            sg, sr = w["scales"]
            run = (lambda a: ref.gemm_i8_requant(a, b.T, lit.EPI_REQUANT_RND, sg, sr)) if ref is not None else \
                  (lambda a: lit.gemm_i8(a, b.T, lit.EPI_REQUANT_RND, sg, sr, nthreads=threads))
            what = "ReferenceGemm<int8> + RequantReluRequant"
        elif dt == "bf16":
            from composable_kernel_amd.host_tensor import uniform_bf16
            b = uniform_bf16((N, K), -1, 1, 2)
            mk = lambda m: uniform_bf16((m, K), -1, 1, 1)
            run = (lambda a: ref.gemm_bf16(a, b.T)) if ref is not None else (lambda a: lit.gemm_bf16(a, b.T, nthreads=threads))
            what = "ReferenceGemm<bhalf_t>"
        else:
            b = uniform_f16((N, K), -1, 1, 2)
            mk = lambda m: uniform_f16((m, K), -1, 1, 1)
            run = (lambda a: ref.gemm_f16(a, b.T)) if ref is not None else (lambda a: lit.gemm_f16(a, b.T, nthreads=threads))
            what = "ReferenceGemm<half_t> (the D-operand functor of the fused variants left out)" if w.get("fused") \
                else "ReferenceGemm<half_t>"
        call = lambda n: run(mk(n))
    elif w["kind"] == "conv":
        C_, K, f, HW, st, pd, nd, dil = w["C"], w["K"], w["f"], w["HW"], w["st"], w["pd"], w.get("ndim", 2), w.get("dil", 1)
        Ho = (HW + 2 * pd - ((f - 1) * dil + 1)) // st + 1
        unit_name, total, per_unit = "images", w["N"], 2.0 * K * Ho ** nd * C_ * f ** nd
        gen = (lambda shp, seed: uniform_int8(shp, -5, 5, seed)) if dt == "i8" else (lambda shp, seed: uniform_f16(shp, -1, 1, seed))
        wt = gen((K, *[f] * nd, C_), 4)
        if ref is not None:
            run = lambda x: ref.convnd_fwd(x, wt, [st] * nd, [dil] * nd, [pd] * nd)
        else:
            run = lambda x: lit.convnd_fwd(x, wt, [st] * nd, [dil] * nd, [pd] * nd)
        what = f"ReferenceConvFwd<{'int8' if dt == 'i8' else 'half_t'}, {nd} spatial dimensions>, PassThrough output functor"
        call = lambda n: run(gen((n, *[HW] * nd, C_), 3))
    else:
        G, M, N, K, O = (w[k] for k in ("G", "M", "N", "K", "O"))
        unit_name, total, per_unit = "batches", G, 2.0 * M * N * (K + O)
        mk3 = lambda g: [uniform_f16(shp, -0.5, 0.5, 5 + j) for j, shp in enumerate([(g, M, K), (g, N, K), (g, N, O)])]
        if w.get("softmax"):
            fn = ref.batched_gemm_softmax_gemm_f16 if ref is not None else lit.batched_gemm_softmax_gemm_f16
            run = lambda a, b0, b1: fn(a, b0.transpose(0, 2, 1), b1, K ** -0.5)
            what = "ReferenceBatchedGemm -> ReferenceSoftmax -> ReferenceBatchedGemm"
        elif ref is not None:
            run = lambda a, b0, b1: ref.batched_gemm_f16(ref.batched_gemm_f16(a, b0.transpose(0, 2, 1)), b1)
            what = "two chained ReferenceBatchedGemm<half_t> (fp16 intermediate)"
        else:
            run = lambda a, b0, b1: lit.batched_gemm_gemm_f16(a, b0.transpose(0, 2, 1), b1, nthreads=threads)
            what = "two chained batched GEMMs (fp16 intermediate)"
        call = lambda n: run(*mk3(n))
    n0 = min(total, 1 if w["kind"] != "gemm" else 8)
    t0 = time.perf_counter()
    call(n0)
    dt0 = max(time.perf_counter() - t0, 1e-4)
    n = int(min(total, max(n0, n0 * seconds / dt0)))
    if n > n0:
        t0 = time.perf_counter()
        call(n)
        dt0 = time.perf_counter() - t0
    return {"value": round(per_unit * n / dt0 / 1e12, 5), "unit": "TOP/s" if dt == "i8" else "TFLOP/s",
            "cores": min(threads, os.cpu_count() or threads) if ref is not None else threads, "kind": kind,
            "host_cores": os.cpu_count(),
            "sample": f"{n} of {total} {unit_name} of the same problem, {what}"
                      + (" compiled in place (oracle/_ref; it starts one thread per host CPU)" if ref is not None
                         else " restated (oracle/ck_oracle.cpp)") + f", {dt0:.1f} s (input generation included)"}


def resnet50_sweep(args):
    """Every layer of the reference's ResNet-50 script through the automatic instance choice: microseconds, rate, the
    fraction of the binding roofline (algorithmic flops against the MFMA peak or algorithmic bytes against HBM,
    whichever is larger) and the instance that ran."""
    from composable_kernel_amd import capi
    L = capi.lib()
    rows = []
    steps, warm = max(16, min(args.steps, 200)), max(3, min(args.warmup, 20))
    print(f"| layer (N = 256) | dtype | op | instance | us | T(FL)OP/s | GB/s | of roofline |\n|---|---|---|---|---|---|---|---|",
          file=sys.stderr)
    for w in resnet50_workloads():
        x = time_workload(w, steps, warm, -1, not args.no_graph, settle_ms=min(args.settle_ms, 100.0))
        op = capi.OP_CONV2D_FWD_I8 if w["dtype"] == "i8" else capi.OP_CONV2D_FWD_F16
        Ho = (w["HW"] + 2 * w["pd"] - w["f"]) // w["st"] + 1
        desc = capi.Conv2dDesc(w["N"], w["K"], w["C"], w["HW"], w["HW"], w["f"], w["f"], Ho, Ho, w["st"], w["st"], 1, 1,
                               w["pd"], w["pd"], w["pd"], w["pd"])
        epi = {None: capi.EPI_REQUANT_RND if w["dtype"] == "i8" else capi.EPI_PASSTHROUGH,
               "bias_relu": capi.EPI_ADD_RELU, "bias_relu_add": capi.EPI_ADD_RELU_ADD}[w["fused"]]
        inst, runs = capi.conv2d_fwd_plan(op, desc, epi, 1 << 30)
        name = L.ckx_instance_name(op, inst).decode()
        frac = max(x["mfma_frac"], x["hbm_frac"])
        row = {"workload": w["name"], "dtype": w["dtype"], "op": "conv_fwd" + ("_" + w["fused"] if w["fused"] else ""),
               "instance": name, "k_runs": runs, "us": round(x["ms"] * 1e3, 2), "value": round(x["tput"], 1),
               "unit": "TOP/s" if w["dtype"] == "i8" else "TFLOP/s", "GB/s": round(x["gbs"], 1), "bound": x["bound"],
               "frac_of_bound": round(frac, 4)}
        if not args.no_cpu:
            row["cpu_baseline"] = cpu_baseline_row(w, min(args.cpu_seconds, 1.0), args.cpu_threads or None)
        rows.append(row)
        geo = f"C{w['C']} K{w['K']} {w['f']}x{w['f']} {w['HW']}^2 s{w['st']} p{w['pd']}"
        print(f"| {geo} | {w['dtype']} | {row['op']} | {name}{' x' + str(runs) + ' K runs' if runs > 1 else ''} | {row['us']} | "
              f"{row['value']} | {row['GB/s']} | {frac:.2f} {x['bound']} |", file=sys.stderr, flush=True)
    print(json.dumps({"metric": "ResNet-50 conv forward layers, N = 256 (script/profile_resnet50.sh of the reference)",
                      "steps": steps, "warmup": warm, "rows": rows}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=300)
    ap.add_argument("--workload", default="fp16_gemm_4096")
    ap.add_argument("--instance", type=int, default=-1)
    ap.add_argument("--all", action="store_true", help="also time every other config (reported under 'also')")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-threads", type=int, default=0, help="threads of the CPU baseline (default: this job's share of the host)")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--settle-ms", type=float, default=300.0,
                    help="least duration of the untimed clock-settling phase before the warm-up launches (0: none)")
    ap.add_argument("--cpu-seconds", type=float, default=2.0,
                    help="CPU time spent on the reference host operator beside every row under 'also' (the headline "
                         "workload's own CPU leg is sized separately)")
    ap.add_argument("--resnet50", action="store_true",
                    help="instead of the headline: the ResNet-50 layers of the reference's whole-network script "
                         "(script/profile_resnet50.sh) at N = 256, fp16 and int8, plain and fused; one JSON line with a "
                         "row per layer, a table on stderr")
    ap.add_argument("--no-clock", action="store_true",
                    help="do not read the engine clock after the timed region (the reading starts rocm-smi as a child "
                         "process, which a counter-collecting profiler around this program does not allow)")
    ap.add_argument("--vendor", action="store_true",
                    help="also time the vendor library on the headline shapes with the same protocol, in the same "
                         "process (torch.matmul for fp16, torch._int_mm for int8), reported under 'vendor'")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one 256 MiB device-to-device copy (a kernel of known traffic, used to "
                         "scale the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this hot path is a single-GPU kernel library; run with --gpus 1 "
              "(a larger problem would shard over independent output tiles, one launch per GPU)", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from composable_kernel_amd import capi
    capi.lib()   # fail loudly if the HIP library is missing

    if args.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
    if args.resnet50:
        return resnet50_sweep(args)
    w = WORKLOADS[args.workload]
    r = time_workload(w, args.steps, args.warmup, args.instance, not args.no_graph, settle_ms=args.settle_ms,
                      from_idle=True, sample_clock=not args.no_clock)
    also = []
    extra = ["int8_requant_gemm_4096"] if args.workload == "fp16_gemm_4096" else []
    if args.all:
        extra = [n for n in WORKLOADS if n != args.workload]
    for n in extra:
        wl = WORKLOADS[n]
        k_steps, k_warm = max(16, args.steps // 2), max(3, args.warmup // 2)
        x = time_workload(wl, k_steps, k_warm, -1, not args.no_graph, settle_ms=args.settle_ms / 2)
        row = {"workload": n, "dtype": x["dtype"], "ms": round(x["ms"], 5),
               "value": round(x["tput"], 2), "unit": "TOP/s" if x["dtype"] == "i8" else "TFLOP/s",
               "GB/s": round(x["gbs"], 1), "bound": x["bound"],
               "frac_of_bound": round(max(x["mfma_frac"], x["hbm_frac"]), 4),
               "settle_launches": x["settle_launches"], "settle_ms": round(x["settle_ms"], 1)}
        if wl["kind"] == "gemm" and x["bound"] == "hbm" and wl["bytes"] < 128e6:
            # the weight matrix fits the Infinity Cache: also time it cold, 8 copies in turn
            cold = time_workload(wl, k_steps - k_steps % 8, k_warm, -1, not args.no_graph, rotate=8,
                                 settle_ms=args.settle_ms / 2)
            row.update({"cold_ms": round(cold["ms"], 5), "cold_GB/s": round(cold["gbs"], 1),
                        "cold_frac_of_bound": round(cold["hbm_frac"], 4)})
        if not args.no_cpu:
            # the reference's host operator on a bounded sample of the same problem, in the same run
            row["cpu_baseline"] = cpu_baseline_row(wl, args.cpu_seconds, args.cpu_threads or None)
        also.append(row)

    unit = "TOP/s" if w["dtype"] == "i8" else "TFLOP/s"
    traffic = MEASURED_TRAFFIC.get(w["name"]) if args.instance < 0 else None
    if r["bound"] == "mfma":
        roof = {"bound": "mfma", "achieved": round(r["tput"], 2), "peak": PEAK[w["dtype"]], "unit": unit,
                "frac": round(r["mfma_frac"], 4), "traffic": traffic}
    else:
        roof = {"bound": "hbm", "achieved": round(r["gbs"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(r["hbm_frac"], 4), "traffic": traffic}
    roof["traffic_source"] = TRAFFIC_SOURCE if traffic is not None else None
    if r.get("sclk_mhz") and r["bound"] == "mfma":
        # the published peak is the rate at 2400 MHz; with toggling operands the power limit holds the engine
        # clock below it, whatever the instruction stream
        mhz = sum(r["sclk_mhz"]) / len(r["sclk_mhz"])
        roof["sclk_mhz_under_load"] = r["sclk_mhz"]
        roof["frac_of_peak_at_that_clock"] = round(r["mfma_frac"] * PEAK_CLOCK_MHZ / mhz, 4)
    idle = _figures(w, r["from_idle_ms"])
    line = {
        "metric": "int8 TOPS & fp16 TFLOPS at 4096^3 on 1 MI355X; % of dtype MFMA peak",
        "value": round(r["tput"], 2), "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(r["wall_ms"], 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": w["dtype"], "data": "synthetic",
        "config": {"workload": w["name"], "layout": "A row-major, B column-major, C row-major",
                   "accumulate": "int32" if w["dtype"] == "i8" else "fp32",
                   "ops_per_step": w["ops"], "algorithmic_bytes_per_step": w["bytes"]},
        "roofline": roof,
        "kernel_ms": round(r["ms"], 5),
        # untimed launches of the same kernel before the warm-up launches, until the GPU has left its idle clocks
        "settle_launches": r["settle_launches"], "settle_ms": round(r["settle_ms"], 1),
        "settle_blocks_us": r["settle_blocks_us"][:12],
        "from_idle": {"protocol": "1 warm-up + 10 timed launches from the idle GPU, no settling "
                                  "(the reference's launch_and_time_kernel)",
                      "kernel_ms": round(r["from_idle_ms"], 5), "value": round(idle["tput"], 2), "unit": unit,
                      "frac": round(max(idle["mfma_frac"], idle["hbm_frac"]), 4)},
        "also": also,
    }
    if args.vendor:
        line["vendor"] = []
        for n in [args.workload] + [x for x in extra if x in ("fp16_gemm_4096", "int8_requant_gemm_4096")]:
            wl = WORKLOADS[n]
            if wl["kind"] != "gemm" or wl.get("G", 1) > 1 or wl.get("fused") or wl["dtype"] not in ("f16", "i8"):
                continue
            # ours again right before the vendor's, so that both see the same clock state of the same box
            ours = time_workload(wl, args.steps, args.warmup, -1, not args.no_graph, settle_ms=args.settle_ms)
            v = time_workload(wl, args.steps, args.warmup, -1, not args.no_graph, settle_ms=args.settle_ms,
                              launch=vendor_launcher(wl))
            line["vendor"].append({"workload": n, "call": "torch.matmul" if wl["dtype"] == "f16" else "torch._int_mm (int32 C)",
                                   "vendor_ms": round(v["ms"], 5), "ours_ms": round(ours["ms"], 5),
                                   "ours_over_vendor": round(ours["ms"] / v["ms"], 4)})
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(w, args.cpu_threads or None)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
