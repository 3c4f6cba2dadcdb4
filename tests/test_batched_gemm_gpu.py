"""GPU parity of the strided batched GEMM (DeviceBatchedGemm, device_batched_gemm.hpp:24-45) through the
C ABI: int8 bit-exact against per-batch reference GEMMs, fp16 against ReferenceBatchedGemm's restatement
within rtol = atol = 1e-2. Shapes follow test/batched_gemm/batched_gemm_fp16.cpp (batch of 3 with ragged
sizes) plus padded batch strides and one weight matrix shared by all batches (BatchStrideB = 0)."""
import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8
from oracle import fast, lit

pytestmark = pytest.mark.gpu

# (G, M, N, K, pad of the A / B / C batch strides in elements, share B)
CASES = [
    (3, 256, 256, 128, (0, 0, 0), False),
    (3, 130, 200, 272, (16, 32, 8), False),
    (64, 64, 64, 64, (0, 0, 0), False),
    (5, 300, 72, 1040, (0, 0, 24), True),
    (2, 17, 130, 4096, (48, 0, 3), False),
]


def _run(op, a_gmk, b_gnk, c_dtype, bs, share_b, c_op=None):
    import torch
    import gpu_util
    G, M, K = a_gmk.shape
    N = b_gnk.shape[1]
    bsa, bsb, bsc = M * K + bs[0], (0 if share_b else N * K + bs[1]), M * N + bs[2]
    da = torch.zeros(G * bsa, dtype=c_dtype, device="cuda")
    db = torch.zeros(max(G * bsb, N * K), dtype=c_dtype, device="cuda")
    for g in range(G):
        da[g * bsa:g * bsa + M * K] = torch.from_numpy(a_gmk[g].ravel()).cuda()
        if not share_b or g == 0:
            db[g * bsb:g * bsb + N * K] = torch.from_numpy(b_gnk[g].ravel()).cuda()
    dc = torch.full((G * bsc,), 77, dtype=c_dtype, device="cuda")
    arg = op.MakeArgumentPointer(da, db, dc, M, N, K, K, K, N, bsa, bsb, bsc, G, None, None, c_op)
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    flat = dc.cpu().numpy()
    out = np.stack([flat[g * bsc:g * bsc + M * N].reshape(M, N) for g in range(G)])
    if bs[2]:
        gaps = np.concatenate([flat[g * bsc + M * N:(g + 1) * bsc] for g in range(G)])
        assert np.all(gaps == 77), "wrote between the C batches"
    return out


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 0, 3, 6])
def test_batched_gemm_int8_bit_exact(case, instance):
    import torch
    G, M, N, K, bs, share_b = case
    a = uniform_int8((G, M, K), -8, 8, 400 + M)
    b = uniform_int8((G, N, K), -8, 8, 401 + N)
    if share_b:
        b[:] = b[0]
    c_op = ck.RequantReluRequant(0.02, 0.4, rounded=True)
    out = _run(ck.DeviceBatchedGemmInt8(instance), a, b, torch.int8, bs, share_b, c_op)
    for g in range(G):
        np.testing.assert_array_equal(out[g], fast.gemm_i8(a[g], b[g].T, lit.EPI_REQUANT_RND, 0.02, 0.4))


@pytest.mark.parametrize("case", CASES[:4])
def test_batched_gemm_fp16(case):
    import torch
    G, M, N, K, bs, share_b = case
    a = uniform_f16((G, M, K), -1, 1, 410 + M)
    b = uniform_f16((G, N, K), -1, 1, 411 + N)
    if share_b:
        b[:] = b[0]
    out = _run(ck.DeviceBatchedGemmF16(), a, b, torch.float16, bs, share_b)
    ref = lit.batched_gemm_f16(a, np.ascontiguousarray(b.transpose(0, 2, 1)))
    bad, max_err = lit.check_err_f16(out, ref, 1e-2, 1e-2)
    assert bad == 0, max_err


def test_batched_gemm_argument_checks():
    L = capi.lib()
    ok = lambda *x: L.ckx_batched_gemm_is_supported(*x)
    assert ok(capi.OP_GEMM_F16, 64, 64, 64, 64, 64, 64, 4096, 4096, 4096, 4, 0, 1, 0, 0, -1) == capi.OK
    assert ok(capi.OP_GEMM_F16, 64, 64, 64, 64, 64, 64, 4096, 4096, 100, 4, 0, 1, 0, 0, -1) == capi.UNSUPPORTED   # C overlap
    # a batch stride of A that is not a whole 16-byte vector: the element-wise instance (and AUTO through it) only
    assert ok(capi.OP_GEMM_F16, 64, 64, 64, 64, 64, 64, 4100, 4096, 4096, 4, 0, 1, 0, 0, 0) == capi.UNSUPPORTED
    assert ok(capi.OP_GEMM_F16, 64, 64, 64, 64, 64, 64, 4100, 4096, 4096, 4, 0, 1, 0, 0, -1) == capi.OK
    assert ok(capi.OP_GEMM_F16, 64, 64, 64, 64, 64, 64, -8, 4096, 4096, 4, 0, 1, 0, 0, -1) == capi.UNSUPPORTED
    assert ok(capi.OP_GEMM_I8, 64, 64, 64, 64, 64, 64, 4096, 4096, 4096, -1, 0, 1, 0, 0, -1) == capi.INVALID_VALUE
    assert ok(capi.OP_GEMM_I8, 16, 64, 64, 64, 64, 64, 4096, 4096, 4096, 4, 0, 1, 0, 0, 9) == capi.UNSUPPORTED     # skinny
