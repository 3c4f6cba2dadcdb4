"""Helpers shared by the GPU parity tests: device buffers come from torch (plumbing only),
every computation goes through the C ABI of libckx.so."""
import numpy as np
import torch

import composable_kernel_amd as ck
from composable_kernel_amd import capi


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def stream():
    return torch.cuda.current_stream().cuda_stream


def gemm_i8(a_mk, b_nk, c_op, instance=capi.INSTANCE_AUTO, ldc=None, time_kernel=False, allow_unsupported=False):
    """A [M,K] row-major, B given as [N,K] (column-major K x N). Returns int8 [M,N] (and ms)."""
    M, K = a_mk.shape
    N = b_nk.shape[0]
    ldc = ldc or N
    da, db = dev(a_mk), dev(b_nk)
    dc = torch.full((M, ldc), 77, dtype=torch.int8, device="cuda")
    op = ck.DeviceGemmInt8(instance)
    arg = op.MakeArgumentPointer(da, db, dc, M, N, K, a_mk.shape[1], b_nk.shape[1], ldc,
                                 ck.PassThrough(), ck.PassThrough(), c_op)
    if allow_unsupported and not op.IsSupportedArgument(arg):
        return None
    assert op.IsSupportedArgument(arg), capi.last_error()
    ms = op.MakeInvokerPointer().Run(arg, ck.StreamConfig(stream(), time_kernel))
    torch.cuda.synchronize()
    out = dc.cpu().numpy()
    if ldc != N:
        assert np.all(out[:, N:] == 77), "wrote outside the C rows"
    return (out[:, :N], ms) if time_kernel else out[:, :N]


def gemm_f16(a_mk, b_nk, instance=capi.INSTANCE_AUTO, time_kernel=False, allow_unsupported=False):
    M, K = a_mk.shape
    N = b_nk.shape[0]
    da, db = dev(a_mk), dev(b_nk)
    dc = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    op = ck.DeviceGemmF16(instance)
    arg = op.MakeArgumentPointer(da, db, dc, M, N, K, K, K, N)
    if allow_unsupported and not op.IsSupportedArgument(arg):
        return None
    assert op.IsSupportedArgument(arg), capi.last_error()
    ms = op.MakeInvokerPointer().Run(arg, ck.StreamConfig(stream(), time_kernel))
    torch.cuda.synchronize()
    out = dc.cpu().numpy()
    return (out, ms) if time_kernel else out


def conv_instance(op, tag):
    """Index of the conv instance of family `op` (capi.OP_CONV2D_FWD_*) whose name contains `tag`."""
    L = capi.lib()
    hits = [i for i in range(L.ckx_num_instances(op)) if tag.encode() in L.ckx_instance_name(op, i)]
    assert len(hits) == 1, (tag, hits)
    return hits[0]


def conv2d_fwd(inp_nhwc, wei_kyxc, strides, dilations, pads, out_op=None, instance=capi.INSTANCE_AUTO,
               right_pads=None):
    N, Hi, Wi, C = inp_nhwc.shape
    K, Y, X, _ = wei_kyxc.shape
    right_pads = right_pads or pads
    Ho = (Hi + pads[0] + right_pads[0] - ((Y - 1) * dilations[0] + 1)) // strides[0] + 1
    Wo = (Wi + pads[1] + right_pads[1] - ((X - 1) * dilations[1] + 1)) // strides[1] + 1
    di, dw = dev(inp_nhwc), dev(wei_kyxc)
    if inp_nhwc.dtype == np.int8:
        do = torch.full((N, Ho, Wo, K), 77, dtype=torch.int8, device="cuda")
        op = ck.DeviceConv2dFwdInt8(instance)
    else:
        do = torch.full((N, Ho, Wo, K), float("nan"), dtype=torch.float16, device="cuda")
        op = ck.DeviceConv2dFwdF16(instance)
    arg = op.MakeArgumentPointer(di, dw, do, N, K, C, [Hi, Wi], [Y, X], [Ho, Wo], list(strides),
                                 list(dilations), list(pads), list(right_pads), None, None, out_op)
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(stream()))
    torch.cuda.synchronize()
    return do.cpu().numpy()


def convnd_fwd(inp, wei, strides, dilations, pads, out_op=None, instance=capi.INSTANCE_AUTO, right_pads=None,
               workspace=False):
    """Channels-last tensors with 1, 2 or 3 spatial dimensions through DeviceConvNdFwd*."""
    nd = inp.ndim - 2
    N, C, K = inp.shape[0], inp.shape[-1], wei.shape[0]
    in_len, filt = list(inp.shape[1:-1]), list(wei.shape[1:-1])
    right_pads = right_pads or pads
    out_len = [(in_len[i] + pads[i] + right_pads[i] - ((filt[i] - 1) * dilations[i] + 1)) // strides[i] + 1
               for i in range(nd)]
    di, dw = dev(inp), dev(wei)
    if inp.dtype == np.int8:
        do = torch.full((N, *out_len, K), 77, dtype=torch.int8, device="cuda")
        op = ck.DeviceConvNdFwdInt8(nd, instance)
    else:
        do = torch.full((N, *out_len, K), float("nan"), dtype=torch.float16, device="cuda")
        op = ck.DeviceConvNdFwdF16(nd, instance)
    arg = op.MakeArgumentPointer(di, dw, do, N, K, C, in_len, filt, out_len, list(strides), list(dilations),
                                 list(pads), list(right_pads), None, None, out_op)
    assert op.IsSupportedArgument(arg), capi.last_error()
    if workspace:
        need = op.GetWorkSpaceSize(arg)
        ws = torch.full((max(need, 16),), 0x7F, dtype=torch.uint8, device="cuda")
        op.SetWorkSpacePointer(arg, ws)
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(stream()))
    torch.cuda.synchronize()
    return do.cpu().numpy()


def gemm_gemm_f16(a_gmk, b0_gnk, b1_gno, instance=capi.INSTANCE_AUTO):
    G, M, K = a_gmk.shape
    N = b0_gnk.shape[1]
    O = b1_gno.shape[2]
    da, db0, db1 = dev(a_gmk), dev(b0_gnk), dev(b1_gno)
    dc = torch.full((G, M, O), float("nan"), dtype=torch.float16, device="cuda")
    op = ck.DeviceBatchedGemmGemmF16(instance)
    arg = op.MakeArgumentPointer(da, db0, db1, dc, M, N, K, O, G, K, K, O, O, M * K, N * K, N * O, M * O)
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(stream()))
    torch.cuda.synchronize()
    return dc.cpu().numpy()
