"""GPU parity: batched fused GEMM-GEMM (fp16) through the C ABI against the CPU oracle
(two chained ReferenceBatchedGemm with an fp16 intermediate). The operator is absent from the
reference snapshot: parity is unpinned by reference vectors, pinned by the oracle's brute-force
and closed-form tests. Tolerance rtol = atol = 1e-2."""
import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8
from oracle import fast, lit

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def _close(out, ref):
    bad, max_err = lit.check_err_f16(out, ref, RTOL, ATOL)
    assert bad == 0, f"{bad} outside tolerance, max err {max_err}"


@pytest.mark.parametrize("shape", [
    # G, M, N, K, O
    (3, 128, 128, 64, 64), (2, 200, 136, 64, 64), (2, 96, 512, 32, 64), (1, 130, 260, 128, 128),
    (2, 64, 72, 40, 24), (5, 16, 8, 8, 8), (1, 256, 256, 96, 128),
])
def test_gemm_gemm_small_shapes(shape):
    import gpu_util
    G, M, N, K, O = shape
    a = uniform_f16((G, M, K), -0.5, 0.5, 900 + M)
    b0_gnk = uniform_f16((G, N, K), -0.5, 0.5, 901 + N)
    b1 = uniform_f16((G, N, O), -0.5, 0.5, 902 + O)
    out = gpu_util.gemm_gemm_f16(a, b0_gnk, b1)
    _close(out, lit.batched_gemm_gemm_f16(a, b0_gnk.transpose(0, 2, 1), b1))


def test_gemm_gemm_closed_form():
    import gpu_util
    G, M, N, K, O = 2, 128, 64, 32, 64
    out = gpu_util.gemm_gemm_f16(np.ones((G, M, K), np.float16), np.ones((G, N, K), np.float16),
                                 np.full((G, N, O), 0.25, np.float16))
    np.testing.assert_array_equal(out, np.full((G, M, O), K * N * 0.25, np.float16))


def test_gemm_gemm_config5():
    """Benchmark configuration 5: batch 64, (512x64)(64x512)(512x64), U[-0.5, 0.5]."""
    import gpu_util
    G, M, N, K, O = 64, 512, 512, 64, 64
    a = uniform_f16((G, M, K), -0.5, 0.5, 910)
    b0_gnk = uniform_f16((G, N, K), -0.5, 0.5, 911)
    b1 = uniform_f16((G, N, O), -0.5, 0.5, 912)
    out = gpu_util.gemm_gemm_f16(a, b0_gnk, b1)
    _close(out, fast.batched_gemm_gemm_f16(a, b0_gnk.transpose(0, 2, 1), b1))
    for g in (0, 63):
        _close(out[g:g + 1], lit.batched_gemm_gemm_f16(a[g:g + 1], b0_gnk[g:g + 1].transpose(0, 2, 1), b1[g:g + 1]))
    # batches are independent: permuting the batch permutes the output
    perm = np.random.default_rng(3).permutation(G)
    out2 = gpu_util.gemm_gemm_f16(a[perm], b0_gnk[perm], b1[perm])
    np.testing.assert_array_equal(out2.view(np.uint16), out[perm].view(np.uint16))


@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 0, 1, 2])
def test_gemm_gemm_config5_integer_operands_bit_exact(instance):
    """Benchmark configuration 5's shape on integers in [-3, 3]: the intermediate (|sum| <= 9 * 64) is exact in fp32
    and in its fp16 rounding, the output sums (|sum| <= 576 * 3 * 512 < 2^24) are exact in fp32 in any order, so the
    fp16 output must equal the rounded exact product bit for bit."""
    import gpu_util
    G, M, N, K, O = 64, 512, 512, 64, 64
    a = uniform_int8((G, M, K), -3, 3, 920).astype(np.float32)
    b0_gnk = uniform_int8((G, N, K), -3, 3, 921).astype(np.float32)
    b1 = uniform_int8((G, N, O), -3, 3, 922).astype(np.float32)
    exact = np.matmul(np.matmul(a, b0_gnk.transpose(0, 2, 1)), b1)
    assert np.abs(exact).max() < 60000
    out = gpu_util.gemm_gemm_f16(a.astype(np.float16), b0_gnk.astype(np.float16), b1.astype(np.float16),
                                 instance=instance)
    np.testing.assert_array_equal(out, exact.astype(np.float16))


def test_gemm_gemm_unsupported():
    import torch
    d = torch.zeros(1 << 16, dtype=torch.float16, device="cuda")
    op = ck.DeviceBatchedGemmGemmF16()
    arg = op.MakeArgumentPointer(d, d, d, d, 64, 64, 256, 64, 1, 256, 256, 64, 64, 0, 0, 0, 0)
    assert not op.IsSupportedArgument(arg)          # K > 128
    with pytest.raises(RuntimeError):
        op.MakeInvokerPointer().Run(arg)
