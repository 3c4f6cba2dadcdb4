"""GPU parity of the split-K plans (C tiles cut into K runs, raw accumulators in a caller
workspace, second pass sums the runs and applies the epilogue). The run count is chosen by the
library; ckx_set_forced_k_runs forces it here so that small problems exercise every path. int8 stays
bit-exact for any split (int32 partial sums); fp16 slices are added in a fixed order."""
import os

import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8
from oracle import fast, lit

pytestmark = pytest.mark.gpu


@pytest.fixture
def force_split():
    def _set(n):
        capi.lib().ckx_set_forced_k_runs(int(n or 0))
    yield _set
    capi.lib().ckx_set_forced_k_runs(0)


def _run_gemm(op, a, b_nk, c_dtype, c_op=None):
    import torch
    import gpu_util
    M, K = a.shape
    N = b_nk.shape[0]
    da, db = gpu_util.dev(a), gpu_util.dev(b_nk)
    dc = torch.zeros((M, N), dtype=c_dtype, device="cuda")
    arg = op.MakeArgumentPointer(da, db, dc, M, N, K, K, K, N, None, None, c_op)
    assert op.IsSupportedArgument(arg)
    need = op.GetWorkSpaceSize(arg)
    ws = torch.full((max(need, 16),), 0x7F, dtype=torch.uint8, device="cuda")   # garbage on purpose
    op.SetWorkSpacePointer(arg, ws)
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))        # idempotent, workspace reusable
    torch.cuda.synchronize()
    return dc.cpu().numpy(), need


@pytest.mark.parametrize("split", [2, 3, 5, 8])
@pytest.mark.parametrize("shape", [(128, 320, 4096), (130, 200, 2064), (300, 72, 1040), (256, 256, 1024)])
@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 0, 3, 6])
def test_int8_gemm_split_k_bit_exact(force_split, split, shape, instance):
    M, N, K = shape
    a = uniform_int8((M, K), -8, 8, 70 + M)
    b_nk = uniform_int8((N, K), -8, 8, 71 + N)
    force_split(split)
    import torch
    out, need = _run_gemm(ck.DeviceGemmInt8(instance), a, b_nk, torch.int8,
                          ck.RequantReluRequant(0.02, 0.4, rounded=True))
    nk = (K + 127) // 128
    if -(-nk // split) * (split - 1) < nk:
        assert need == split * M * N * 4        # the forced split was taken
    np.testing.assert_array_equal(out, fast.gemm_i8(a, b_nk.T, lit.EPI_REQUANT_RND, 0.02, 0.4))


@pytest.mark.parametrize("split", [2, 4])
def test_fp16_gemm_split_k(force_split, split):
    import torch
    M, N, K = 136, 264, 2056
    a = uniform_f16((M, K), -1, 1, 72)
    b_nk = uniform_f16((N, K), -1, 1, 73)
    force_split(split)
    out, need = _run_gemm(ck.DeviceGemmF16(), a, b_nk, torch.float16)
    assert need == split * M * N * 4
    bad, max_err = lit.check_err_f16(out, lit.gemm_f16(a, b_nk.T), 1e-2, 1e-2)
    assert bad == 0, max_err
    out2, _ = _run_gemm(ck.DeviceGemmF16(), a, b_nk, torch.float16)
    np.testing.assert_array_equal(out.view(np.uint16), out2.view(np.uint16))   # fixed summation order


def test_split_k_without_workspace_falls_back(force_split):
    import torch
    import gpu_util
    M, N, K = 128, 256, 4096
    a = uniform_int8((M, K), -8, 8, 74)
    b_nk = uniform_int8((N, K), -8, 8, 75)
    force_split(4)
    out = gpu_util.gemm_i8(a, b_nk, ck.PassThrough())        # no workspace attached
    np.testing.assert_array_equal(out, fast.gemm_i8(a, b_nk.T))


@pytest.mark.parametrize("dtype", ["int8", "fp16"])
def test_conv2d_split_k(force_split, dtype):
    import torch
    import gpu_util
    N, C, K, HW = 3, 64, 96, 7
    s, d, p = (1, 1), (1, 1), (1, 1)
    force_split(3)
    if dtype == "int8":
        inp = uniform_int8((N, HW, HW, C), -5, 5, 76)
        wei = uniform_int8((K, 3, 3, C), -5, 5, 77)
        op, tdt = ck.DeviceConv2dFwdInt8(), torch.int8
        out_op = ck.RequantReluRequant(0.05, 0.7, rounded=True)
    else:
        inp = uniform_f16((N, HW, HW, C), -1, 1, 76)
        wei = uniform_f16((K, 3, 3, C), -1, 1, 77)
        op, tdt = ck.DeviceConv2dFwdF16(), torch.float16
        out_op = None
    di, dw = gpu_util.dev(inp), gpu_util.dev(wei)
    do = torch.zeros((N, HW, HW, K), dtype=tdt, device="cuda")
    arg = op.MakeArgumentPointer(di, dw, do, N, K, C, [HW, HW], [3, 3], [HW, HW], [1, 1], [1, 1], [1, 1], [1, 1],
                                 None, None, out_op)
    need = op.GetWorkSpaceSize(arg)
    assert need == 3 * N * HW * HW * K * 4
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    op.SetWorkSpacePointer(arg, ws)
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    if dtype == "int8":
        np.testing.assert_array_equal(
            do.cpu().numpy(), lit.conv2d_fwd(inp, wei, s, d, p, epi=lit.EPI_REQUANT_RND, scale_gemm=0.05, scale_relu=0.7))
    else:
        bad, max_err = lit.check_err_f16(do.cpu().numpy(), lit.conv2d_fwd(inp, wei, s, d, p), 1e-2, 1e-2)
        assert bad == 0, max_err


@pytest.mark.parametrize("shape", [(8, 10300, 256), (9, 10300, 256), (16, 5200, 192), (16, 1000, 320), (17, 10300, 128),
                                   (32, 5200, 256), (33, 10300, 128), (48, 700, 4096), (64, 10304, 192), (65, 700, 2048),
                                   # few columns under a long K (tile kernel with a K split when the workspace is there),
                                   # many columns under up to 4 rows (wide skinny instance), 33..64 rows at K = 4096
                                   (8, 1024, 8192), (16, 528, 16384), (32, 2048, 8192), (24, 4096, 8208), (4, 16384, 1024),
                                   (1, 16400, 512), (48, 4096, 4096), (64, 2048, 8192)])
def test_auto_instance_few_rows_routing_bit_exact(shape):
    """Automatic choice for few-row problems: narrow / wide skinny instances up to 32 rows, skinny or
    tile kernel (with a K split when the workspace is there) up to 64 rows. Every route must give
    the reference's bits, with and without a workspace."""
    import torch
    import gpu_util
    M, N, K = shape
    a = uniform_int8((M, K), -8, 8, 90 + M)
    b_nk = uniform_int8((N, K), -8, 8, 91 + N)
    c_op = ck.RequantReluRequant(0.02, 0.4, rounded=True)
    ref = fast.gemm_i8(a, b_nk.T, lit.EPI_REQUANT_RND, 0.02, 0.4)
    out, _ = _run_gemm(ck.DeviceGemmInt8(), a, b_nk, torch.int8, c_op)
    np.testing.assert_array_equal(out, ref)
    np.testing.assert_array_equal(gpu_util.gemm_i8(a, b_nk, c_op), ref)       # no workspace
    af, bf = uniform_f16((M, K), -1, 1, 92 + M), uniform_f16((N, K), -1, 1, 93 + N)
    outf, _ = _run_gemm(ck.DeviceGemmF16(), af, bf, torch.float16)
    reff = fast.gemm_f16(af, bf.T)
    assert np.all(np.abs(outf.astype(np.float32) - reff.astype(np.float32)) <= 1e-2 + 1e-2 * np.abs(reff.astype(np.float32)))


def _run_splitk(op, a, b_nk, c_dtype, kbatch, c_op=None, give_workspace=True):
    import torch
    import gpu_util
    M, K = a.shape
    N = b_nk.shape[0]
    da, db = gpu_util.dev(a), gpu_util.dev(b_nk)
    dc = torch.zeros((M, N), dtype=c_dtype, device="cuda")
    arg = op.MakeArgumentPointer(da, db, dc, M, N, K, K, K, N, None, None, c_op, kbatch)
    if not op.IsSupportedArgument(arg):
        return None, 0
    need = op.GetWorkSpaceSize(arg)
    if give_workspace:
        ws = torch.full((max(need, 16),), 0x7F, dtype=torch.uint8, device="cuda")
        op.SetWorkSpacePointer(arg, ws)
    st = op._launch(arg, gpu_util.stream())
    torch.cuda.synchronize()
    return (dc.cpu().numpy() if st == 0 else st), need


@pytest.mark.parametrize("kbatch", [1, 2, 4, 8])
@pytest.mark.parametrize("shape", [(128, 320, 4096), (130, 200, 2064), (16, 64, 256)])
def test_device_gemm_splitk_kbatch_argument(shape, kbatch):
    """DeviceGemmSplitK's KBatch (device_gemm_splitk.hpp:14-39): the caller fixes the number of K runs.
    int8 is bit-identical to the unsplit result for every KBatch; fp16 within tolerance; a K with
    fewer 128-byte tiles than KBatch uses fewer runs."""
    import torch
    M, N, K = shape
    a = uniform_int8((M, K), -8, 8, 170 + M)
    b_nk = uniform_int8((N, K), -8, 8, 171 + N)
    out, need = _run_splitk(ck.DeviceGemmSplitKInt8(), a, b_nk, torch.int8, kbatch,
                            ck.RequantReluRequant(0.02, 0.4, rounded=True))
    nk = (K + 127) // 128
    runs = next(sp for sp in range(min(kbatch, 8), 0, -1) if sp == 1 or -(-nk // sp) * (sp - 1) < nk)
    assert need == (runs * M * N * 4 if runs > 1 else 0)
    np.testing.assert_array_equal(out, fast.gemm_i8(a, b_nk.T, lit.EPI_REQUANT_RND, 0.02, 0.4))
    af, bf = uniform_f16((M, K // 2), -1, 1, 172 + M), uniform_f16((N, K // 2), -1, 1, 173 + N)
    outf, _ = _run_splitk(ck.DeviceGemmSplitKF16(3), af, bf, torch.float16, kbatch)
    bad, max_err = lit.check_err_f16(outf, fast.gemm_f16(af, bf.T), 1e-2, 1e-2)
    assert bad == 0, max_err


def test_device_gemm_splitk_rejects_missing_workspace_and_bad_kbatch():
    import torch
    a = uniform_int8((64, 1024), -8, 8, 1)
    b_nk = uniform_int8((64, 1024), -8, 8, 2)
    st, need = _run_splitk(ck.DeviceGemmSplitKInt8(), a, b_nk, torch.int8, 4, ck.PassThrough(), give_workspace=False)
    assert need == 4 * 64 * 64 * 4 and st == capi.INVALID_VALUE and "workspace" in capi.last_error()
    out, _ = _run_splitk(ck.DeviceGemmSplitKInt8(), a, b_nk, torch.int8, 9, ck.PassThrough())
    assert out is None
    out, _ = _run_splitk(ck.DeviceGemmSplitKInt8(capi.lib().ckx_num_instances(capi.OP_GEMM_SPLITK)), a, b_nk,
                         torch.int8, 2, ck.PassThrough())
    assert out is None      # a skinny instance
