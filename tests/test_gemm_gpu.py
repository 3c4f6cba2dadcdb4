"""GPU parity: int8 / fp16 GEMM through the C ABI against the CPU oracle.

Mirrors the reference's own integration tests: test/gemm/gemm_int8.cpp and gemm_fp16.cpp run
every instance at 1024^3 against ReferenceGemm (test/gemm/gemm_util.hpp:123-240), and
example 14 checks the fused requant epilogue. int8 results must be bit-exact; fp16 within
rtol = atol = 1e-2 of the fp32-accumulated reference (the reference's own check_err default
for half, 1e-3 / 1e-3, is also reported where it holds).
"""
import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8
from oracle import fast, lit

pytestmark = pytest.mark.gpu

N_INSTANCES = 19        # tile instances, the skinny (few-row) and weight-streaming instances, the element-wise (padding) instance
SKINNY_MAX_M = {9: 16, 10: 32, 11: 64, 12: 16, 13: 16, 14: 16, 15: 32, 16: 32, 17: 128}
RTOL = ATOL = 1e-2

EPILOGUES = {
    "passthrough": (ck.PassThrough(), lit.EPI_PASSTHROUGH, 1.0, 1.0),
    "ck_ex14": (ck.RequantReluRequant(0.03, 1.0), lit.EPI_REQUANT_CK, 0.03, 1.0),
    "rounded_cfg1": (ck.RequantReluRequant(0.5, 0.03, rounded=True), lit.EPI_REQUANT_RND, 0.5, 0.03),
    "rounded_cfg3": (ck.RequantReluRequant(0.02, 0.4, rounded=True), lit.EPI_REQUANT_RND, 0.02, 0.4),
}


def _assert_f16_close(out, ref, rtol=RTOL, atol=ATOL):
    bad, max_err = lit.check_err_f16(out, ref, rtol, atol)
    assert bad == 0, f"{bad} elements outside |o-r| <= {atol} + {rtol}|r| (max err {max_err})"


@pytest.mark.parametrize("epi", list(EPILOGUES))
def test_int8_gemm_config1_1024_cubed_bit_exact(epi):
    """Benchmark configuration 1: M=N=K=1024, int8 in [-5,5], literal ReferenceGemm oracle."""
    import gpu_util
    c_op, kind, sg, sr = EPILOGUES[epi]
    a = uniform_int8((1024, 1024), -5, 5, 0xC0FFEE)
    b_nk = uniform_int8((1024, 1024), -5, 5, 0xC0FFEE + 1)
    out = gpu_util.gemm_i8(a, b_nk, c_op)
    want = lit.gemm_i8(a, b_nk.T, kind, sg, sr)
    np.testing.assert_array_equal(out, want)
    if kind != lit.EPI_PASSTHROUGH:
        assert out.max() > 0  # the epilogue is not degenerate on this data


def test_instance_count_matches_the_library():
    assert capi.lib().ckx_num_instances(capi.OP_GEMM_I8) == N_INSTANCES
    assert capi.lib().ckx_num_instances(capi.OP_GEMM_F16) == N_INSTANCES


@pytest.mark.parametrize("instance", range(N_INSTANCES))
@pytest.mark.parametrize("shape", [(256, 256, 256), (300, 200, 128), (17, 130, 1040), (1, 64, 16), (513, 80, 4096),
                                   (16, 208, 4096), (5, 48, 11008), (33, 100, 2064), (64, 16, 80)])
def test_int8_gemm_every_instance_ragged_shapes(instance, shape):
    """Every instance on every shape, as test/gemm/gemm_util.hpp:123-240 does; an instance that
    does not support a shape must say so (gemm_util.hpp:235-238) instead of computing."""
    import gpu_util
    M, N, K = shape
    a = uniform_int8((M, K), -8, 8, 11 + M)
    b_nk = uniform_int8((N, K), -8, 8, 13 + N)
    c_op, kind, sg, sr = EPILOGUES["rounded_cfg3"]
    out = gpu_util.gemm_i8(a, b_nk, c_op, instance=instance, ldc=N + 16, allow_unsupported=True)
    if out is None:
        assert instance in SKINNY_MAX_M and M > SKINNY_MAX_M[instance]
        return
    np.testing.assert_array_equal(out, fast.gemm_i8(a, b_nk.T, kind, sg, sr))
    out = gpu_util.gemm_i8(a, b_nk, ck.PassThrough(), instance=instance)
    np.testing.assert_array_equal(out, fast.gemm_i8(a, b_nk.T))


def test_int8_gemm_full_range_values_wrap_like_the_reference():
    import gpu_util
    a = uniform_int8((96, 512), -128, 127, 5)
    b_nk = uniform_int8((72, 512), -128, 127, 6)
    out = gpu_util.gemm_i8(a, b_nk, ck.PassThrough())
    np.testing.assert_array_equal(out, lit.gemm_i8(a, b_nk.T))   # int32 accumulate, low byte


def test_int8_gemm_padded_strides():
    import gpu_util
    M, N, K = 130, 96, 200 + 8   # K multiple of 16
    abuf = uniform_int8((M, K + 48), -5, 5, 21)
    bbuf = uniform_int8((N, K + 16), -5, 5, 22)
    a, b_nk = abuf[:, :K], bbuf[:, :K]
    import torch
    da, db = gpu_util.dev(abuf), gpu_util.dev(bbuf)
    dc = torch.zeros((M, N), dtype=torch.int8, device="cuda")
    op = ck.DeviceGemmInt8()
    arg = op.MakeArgumentPointer(da, db, dc, M, N, K, K + 48, K + 16, N, None, None,
                                 ck.RequantReluRequant(0.5, 0.03, rounded=True))
    assert op.IsSupportedArgument(arg)
    op.MakeInvokerPointer().Run(arg)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(dc.cpu().numpy(), lit.gemm_i8(a, b_nk.T, lit.EPI_REQUANT_RND, 0.5, 0.03))


def test_epilogue_exhaustive_through_the_gemm():
    """Drive the GEMM's own epilogue with every accumulator in [-2^15, 2^15) x a few scales:
    A = [hi, lo, 1...] B = [[128], [1], ...] style decomposition acc = 127*h + l."""
    import gpu_util
    # acc(m, n) = sum_k a[m,k] b[n,k] with K = 16: use a[m,:2] = (m_hi, m_lo), b[n,:2] = (127, 1) etc.
    vals = np.arange(-16000, 16000, dtype=np.int64)
    hi, lo = np.divmod(vals, 127)          # vals = 127*hi + lo, 0 <= lo < 127, |hi| <= 126
    M = len(vals)
    a = np.zeros((M, 16), np.int8)
    a[:, 0], a[:, 1] = hi, lo
    b_nk = np.zeros((16, 16), np.int8)
    b_nk[:, 0], b_nk[:, 1] = 127, 1
    b_nk[1, 0], b_nk[1, 1] = -127, -1      # second column: negated accumulators
    acc = fast.gemm_i8_acc(a, b_nk.T)
    np.testing.assert_array_equal(acc[:, 0], vals)
    for name, (c_op, kind, sg, sr) in EPILOGUES.items():
        out = gpu_util.gemm_i8(a, b_nk, c_op)
        want = np.array([[lit.epilogue_i8(int(v), kind, sg, sr) for v in row] for row in acc[:, :2]], np.int8)
        np.testing.assert_array_equal(out[:, :2], want, err_msg=name)


def test_int8_gemm_unsupported_arguments_are_refused():
    import gpu_util
    import torch
    op = ck.DeviceGemmInt8()
    d = torch.zeros(1 << 16, dtype=torch.int8, device="cuda")
    # K not a multiple of 16 bytes: the vectorised instances refuse (as the reference's Default-specialisation
    # instances do), the element-wise instance and the automatic choice take it (its KPadding instances)
    for instance in range(N_INSTANCES - 1):
        fast = ck.DeviceGemmInt8(instance)
        arg = fast.MakeArgumentPointer(d, d, d, 16, 64, 100, 100, 100, 64)
        assert not fast.IsSupportedArgument(arg)
        with pytest.raises(RuntimeError):
            fast.MakeInvokerPointer().Run(arg)
    assert op.IsSupportedArgument(op.MakeArgumentPointer(d, d, d, 64, 64, 100, 100, 100, 64))
    # a leading dimension below the row length
    assert not op.IsSupportedArgument(op.MakeArgumentPointer(d, d, d, 64, 64, 100, 99, 100, 64))
    # column-major C is not built (nor is it in the reference's instance lists)
    op2 = ck.DeviceGemmInt8(CLayout=ck.ColumnMajor)
    assert not op2.IsSupportedArgument(op2.MakeArgumentPointer(d, d, d, 64, 64, 64, 64, 64, 64))
    # empty problem is a no-op
    arg = op.MakeArgumentPointer(d, d, d, 0, 64, 64, 64, 64, 64)
    assert op.IsSupportedArgument(arg)
    op.MakeInvokerPointer().Run(arg)
    torch.cuda.synchronize()


@pytest.mark.parametrize("instance", range(N_INSTANCES))
@pytest.mark.parametrize("shape", [(260, 200, 328), (16, 72, 1032), (40, 24, 520), (1, 16, 8)])
def test_fp16_gemm_every_instance_vs_literal_oracle(instance, shape):
    import gpu_util
    M, N, K = shape
    a = uniform_f16((M, K), -1, 1, 31)
    b_nk = uniform_f16((N, K), -1, 1, 32)
    out = gpu_util.gemm_f16(a, b_nk, instance=instance, allow_unsupported=True)
    if out is None:
        assert instance in SKINNY_MAX_M and M > SKINNY_MAX_M[instance]
        return
    _assert_f16_close(out, lit.gemm_f16(a, b_nk.T))


def test_fp16_gemm_closed_forms():
    import gpu_util
    M, N, K = 64, 128, 512
    out = gpu_util.gemm_f16(np.ones((M, K), np.float16), np.ones((N, K), np.float16))
    np.testing.assert_array_equal(out, np.full((M, N), K, np.float16))
    # identity B copies A
    a = uniform_f16((96, 128), -1, 1, 33)
    out = gpu_util.gemm_f16(a, np.eye(128, dtype=np.float16))
    np.testing.assert_array_equal(out, a)


def test_fp16_gemm_config2_4096_cubed_within_tolerance():
    """Benchmark configuration 2 (fp16, 4096^3). Full output against the fp32 BLAS form, a sample of rows against the
    literal sequential-k oracle."""
    import gpu_util
    M = N = K = 4096
    a = uniform_f16((M, K), -1, 1, 41)
    b_nk = uniform_f16((N, K), -1, 1, 42)
    out = gpu_util.gemm_f16(a, b_nk)
    _assert_f16_close(out, fast.gemm_f16(a, b_nk.T))
    rows = np.random.default_rng(0).choice(M, 24, replace=False)
    _assert_f16_close(out[rows], lit.gemm_f16(a[rows], b_nk.T))
    bad_strict, _ = lit.check_err_f16(out[rows], lit.gemm_f16(a[rows], b_nk.T), 1e-3, 1e-3)
    print("fp16 4096^3: elements outside the reference's 1e-3/1e-3 on sampled rows:", bad_strict)


def test_fp16_gemm_4096_cubed_integer_operands_bit_exact():
    """The reference profiler's initialisation 1 (integers in [-5, 5]) at the metric shape: every partial sum is an
    integer below 2^24 in magnitude (|sum| <= 25 * 4096), so fp32 accumulation is exact in any order and the fp16
    output must equal the rounded exact product bit for bit -- a full-size check that no tolerance can hide an
    indexing mistake behind."""
    import gpu_util
    M = N = K = 4096
    a = uniform_int8((M, K), -5, 5, 61).astype(np.float32)
    b_nk = uniform_int8((N, K), -5, 5, 62).astype(np.float32)
    exact = a @ b_nk.T                      # exact: integers below 2^24 in fp32
    assert np.abs(exact).max() < 60000      # inside fp16's range
    out = gpu_util.gemm_f16(a.astype(np.float16), b_nk.astype(np.float16))
    np.testing.assert_array_equal(out, exact.astype(np.float16))


def test_int8_gemm_4096_cubed_bit_exact():
    """Metric shape: full output against the exact fp32-BLAS form, sampled rows against the
    literal oracle."""
    import gpu_util
    M = N = K = 4096
    a = uniform_int8((M, K), -5, 5, 51)
    b_nk = uniform_int8((N, K), -5, 5, 52)
    c_op, kind, sg, sr = EPILOGUES["rounded_cfg1"]
    out = gpu_util.gemm_i8(a, b_nk, c_op)
    np.testing.assert_array_equal(out, fast.gemm_i8(a, b_nk.T, kind, sg, sr))
    rows = np.random.default_rng(1).choice(M, 16, replace=False)
    np.testing.assert_array_equal(out[rows], lit.gemm_i8(a[rows], b_nk.T, kind, sg, sr))


@pytest.mark.parametrize("M", [1, 16, 128, 4096])
@pytest.mark.parametrize("NK", [(11008, 4096), (4096, 11008)])
def test_int8_gemm_config3_llm_shapes_bit_exact(M, NK):
    """Benchmark configuration 3: tokens x N x K, int8 in [-8,8], scales 0.02 / 0.4, rounded mode."""
    import gpu_util
    N, K = NK
    a = uniform_int8((M, K), -8, 8, 61 + M)
    b_nk = uniform_int8((N, K), -8, 8, 62 + N)
    c_op, kind, sg, sr = EPILOGUES["rounded_cfg3"]
    out = gpu_util.gemm_i8(a, b_nk, c_op)
    np.testing.assert_array_equal(out, fast.gemm_i8(a, b_nk.T, kind, sg, sr))
    rows = np.random.default_rng(2).choice(M, min(M, 4), replace=False)
    np.testing.assert_array_equal(out[rows], lit.gemm_i8(a[rows], b_nk.T, kind, sg, sr))
