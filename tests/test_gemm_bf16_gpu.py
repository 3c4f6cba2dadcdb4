"""GPU parity of the bf16 GEMM (DeviceGemm<..., bhalf_t x3, PassThrough x3>) through the C ABI: fp32
accumulation, one round-to-nearest-even conversion. Tolerance rtol = atol = 1e-2 on the values
(one bf16 ulp is at most 0.8 %); exact where the result is a small integer."""
import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_bf16
from oracle import fast, lit

pytestmark = pytest.mark.gpu


def _gemm(a, b_nk, instance=capi.INSTANCE_AUTO, workspace=False):
    import torch
    import gpu_util
    M, K = a.shape
    N = b_nk.shape[0]
    da = torch.from_numpy(a.view(np.int16)).cuda()
    db = torch.from_numpy(b_nk.view(np.int16)).cuda()
    dc = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")   # NaN pattern
    op = ck.DeviceGemmBF16(instance)
    arg = op.MakeArgumentPointer(da, db, dc, M, N, K, K, K, N)
    if not op.IsSupportedArgument(arg):
        return None
    if workspace:
        ws = torch.full((max(op.GetWorkSpaceSize(arg), 16),), 0x7F, dtype=torch.uint8, device="cuda")
        op.SetWorkSpacePointer(arg, ws)
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    return dc.cpu().numpy().view(np.uint16)


def _close(out, ref):
    o, r = fast.bf16_to_f32(out), fast.bf16_to_f32(ref)
    assert np.all(np.isfinite(o))
    assert np.all(np.abs(o - r) <= 1e-2 + 1e-2 * np.abs(r)), np.abs(o - r).max()


@pytest.mark.parametrize("shape", [(256, 256, 256), (300, 200, 128), (17, 130, 1040), (1, 64, 16), (513, 80, 4096),
                                   (16, 208, 4096), (33, 100, 2064)])
@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 0, 2, 5, 8, 9, 13])
def test_bf16_gemm_against_the_oracle(shape, instance):
    M, N, K = shape
    a = uniform_bf16((M, K), -1, 1, 600 + M)
    b_nk = uniform_bf16((N, K), -1, 1, 601 + N)
    out = _gemm(a, b_nk, instance)
    if out is None:
        assert instance >= 9       # a skinny instance with fewer rows than M
        return
    _close(out, lit.gemm_bf16(a, b_nk.T))


def test_bf16_gemm_exact_small_integers_and_tie():
    """Ones: every entry is K. K = 257 is not representable (8 significant bits): the tie goes to 256."""
    one = np.uint16(0x3F80)
    a = np.full((40, 264), one, np.uint16)
    a[:, 257:] = 0
    b_nk = np.full((48, 264), one, np.uint16)
    out = _gemm(a, b_nk)
    assert np.all(fast.bf16_to_f32(out) == 256.0)
    a[:, 192:] = 0
    assert np.all(fast.bf16_to_f32(_gemm(a, b_nk)) == 192.0)


def test_bf16_gemm_full_size_and_split_k(force_k_runs):
    a = uniform_bf16((1024, 2048), -1, 1, 31)
    b_nk = uniform_bf16((768, 2048), -1, 1, 32)
    ref = fast.gemm_bf16(a, b_nk.T)
    _close(_gemm(a, b_nk), ref)
    force_k_runs(4)
    _close(_gemm(a, b_nk, workspace=True), ref)


def test_bf16_gemm_4096_cubed_integer_operands_bit_exact():
    """Integers in [-5, 5] at the metric shape: fp32 accumulation is exact in any order (|sum| <= 25 * 4096 < 2^24), so
    the bf16 output must be the round-to-nearest-even of the exact product, bit for bit."""
    from composable_kernel_amd.host_tensor import uniform_int8
    M = N = K = 4096
    a = uniform_int8((M, K), -5, 5, 41).astype(np.float32)
    b_nk = uniform_int8((N, K), -5, 5, 42).astype(np.float32)
    exact = a @ b_nk.T
    out = _gemm(fast.f32_to_bf16(a), fast.f32_to_bf16(b_nk))
    np.testing.assert_array_equal(out, fast.f32_to_bf16(exact))


def test_bf16_gemm_has_no_fused_epilogue():
    op = ck.DeviceGemmBF16()
    arg = op.MakeArgumentPointer(0, 0, 0, 64, 64, 64, 64, 64, 64, None, None, ck.RequantReluRequant(1, 1))
    assert not op.IsSupportedArgument(arg)
    assert capi.lib().ckx_num_instances(capi.OP_GEMM_BF16) == capi.lib().ckx_num_instances(capi.OP_GEMM_F16)
    assert b"bf16" in capi.lib().ckx_instance_name(capi.OP_GEMM_BF16, 0)
