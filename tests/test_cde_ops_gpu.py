"""GPU parity of the scaled and GELU CDE operations of the fp16 DeviceGemmMultipleD, through the C ABI:

  * Bilinear        E = half(alpha * (A*B) + beta * D)         (example 02, profiler command gemm_bilinear)
  * AddAddFastGelu  E = half(fast_gelu(A*B + D0 + D1))         (example 04, profiler command gemm_add_add_fastgelu)

against the CPU oracle (element-by-element form on small problems, BLAS form on larger ones), rtol = atol = 1e-2 (the
fp16 bar of the reference's check_err), plus cases whose result is exact, so that a wrong order of operations, a rounding
too many or swapped operands show. Every instance family runs them: the tile kernels (own epilogue variants), the skinny
and element-wise kernels, and the second pass of a K split.
"""
import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_f16
from oracle import fast, lit

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2
LAYOUTS = {"mk_nk": (ck.RowMajor, ck.ColumnMajor), "mk_kn": (ck.RowMajor, ck.RowMajor),
           "km_kn": (ck.ColumnMajor, ck.RowMajor), "km_nk": (ck.ColumnMajor, ck.ColumnMajor)}


def _instance(tag):
    """'generic': the element-wise instance, the last of the family"""
    if tag != "generic":
        return tag
    L = capi.lib()
    n = L.ckx_num_instances(capi.OP_GEMM_F16)
    assert b"Generic" in L.ckx_instance_name(capi.OP_GEMM_F16, n - 1)
    return n - 1


def _close(out, ref):
    bad, max_err = lit.check_err_f16(out, ref, RTOL, ATOL)
    assert bad == 0, f"{bad} outside tolerance, max err {max_err}"


def _run(a_mk, b_kn, ds, strides, functor, instance=capi.INSTANCE_AUTO, layout="mk_nk", lde=None, workspace=False,
         allow_unsupported=False):
    import torch
    import gpu_util
    M, K = a_mk.shape
    N = b_kn.shape[1]
    al, bl = LAYOUTS[layout]
    a_st = np.ascontiguousarray(a_mk.T) if al is ck.ColumnMajor else np.ascontiguousarray(a_mk)
    b_st = np.ascontiguousarray(b_kn) if bl is ck.RowMajor else np.ascontiguousarray(b_kn.T)
    lde = lde or N
    da, db = gpu_util.dev(a_st), gpu_util.dev(b_st)
    dds = [gpu_util.dev(d) for d in ds]
    de = torch.full((M, lde), 77.0, dtype=torch.float16, device="cuda")
    op = ck.DeviceGemmMultipleDF16(instance, ALayout=al, BLayout=bl)
    arg = op.MakeArgumentPointer(da, db, dds, de, M, N, K, a_st.shape[1], b_st.shape[1], strides, lde, None, None,
                                 functor)
    if allow_unsupported and not op.IsSupportedArgument(arg):
        return None
    assert op.IsSupportedArgument(arg), capi.last_error()
    if workspace:
        need = op.GetWorkSpaceSize(arg)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        op.SetWorkSpacePointer(arg, ws, need)
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    out = de.cpu().numpy()
    assert np.all(out[:, N:] == 77.0), "wrote outside the E rows"
    return out[:, :N]


SHAPES = [(256, 256, 256), (300, 200, 128), (17, 130, 1040), (5, 48, 4096), (64, 100, 80), (513, 88, 512)]
INSTANCES = [capi.INSTANCE_AUTO, 0, 2, 5, 9, 11, 13]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("instance", INSTANCES)
def test_gemm_bilinear_like_example_02(shape, instance):
    """D a full [M,N] tensor with a padded row stride (example 02's StrideD), and one broadcast row."""
    M, N, K = shape
    a = uniform_f16((M, K), -1, 1, 900 + M)
    b_kn = uniform_f16((K, N), -1, 1, 901 + N)
    d = uniform_f16((M, N + 8), -3, 3, 902 + N)
    out = _run(a, b_kn, [d], [N + 8], ck.Bilinear(0.75, -1.5), instance, allow_unsupported=True)
    if out is None:
        assert instance >= 9     # a skinny instance with fewer rows than M
        return
    _close(out, fast.gemm_f16_bilinear(a, b_kn, d[:, :N], 0.75, -1.5))
    row = uniform_f16((1, N), -3, 3, 903 + N)
    _close(_run(a, b_kn, [row], [0], ck.Bilinear(-2.0, 0.5), instance, lde=N + 24),
           fast.gemm_f16_bilinear(a, b_kn, row, -2.0, 0.5))


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("instance", INSTANCES)
def test_gemm_add_add_fastgelu_like_example_04(shape, instance):
    """D0 a bias row (stride 0) and D1 a full tensor, as example 04 passes them; then both full tensors."""
    M, N, K = shape
    a = uniform_f16((M, K), -0.5, 0.5, 950 + M)
    b_kn = uniform_f16((K, N), -0.5, 0.5, 951 + N)
    d0 = uniform_f16((1, N), -2, 2, 952 + N)
    d1 = uniform_f16((M, N + 8), -2, 2, 953 + N)
    out = _run(a, b_kn, [d0, d1], [0, N + 8], ck.AddAddFastGelu(), instance, allow_unsupported=True)
    if out is None:
        assert instance >= 9
        return
    ref = fast.gemm_f16_add_add_fastgelu(a, b_kn, d0, d1[:, :N])
    _close(out, ref)
    assert (out < 0).any() and (out > 0.5).any()
    d0_full = uniform_f16((M, N), -2, 2, 954 + N)
    _close(_run(a, b_kn, [d0_full, d1], [N, N + 8], ck.AddAddFastGelu(), instance, lde=N + 8),
           fast.gemm_f16_add_add_fastgelu(a, b_kn, d0_full, d1[:, :N]))


@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 0, 4, 9, 13, "generic"])
def test_small_problems_against_the_element_by_element_oracle(instance):
    instance = _instance(instance)
    M, N, K = 13, 40, 96
    a = uniform_f16((M, K), -1, 1, 1000)
    b_kn = uniform_f16((K, N), -1, 1, 1001)
    d0, d1 = uniform_f16((M, N), -3, 3, 1002), uniform_f16((M, N), -2, 2, 1003)
    _close(_run(a, b_kn, [d0], [N], ck.Bilinear(1.25, 0.5), instance), lit.gemm_f16_bilinear(a, b_kn, d0, 1.25, 0.5))
    _close(_run(a, b_kn, [d0, d1], [N, N], ck.AddAddFastGelu(), instance),
           lit.gemm_f16_add_add_fastgelu(a, b_kn, d0, d1))


@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 0, 3, 9, 13, "generic"])
def test_bilinear_exact_cases(instance):
    """K = 2049 ones: acc = 2049. alpha = beta = 1 with d = 1 stores 2050 (rounding C to fp16 first would store 2048);
    alpha = 2, beta = -3 in integers; alpha = 0, beta = 1 returns D bit for bit; alpha = 1, beta = 0 is the plain
    GEMM of the same instance bit for bit."""
    import gpu_util
    instance = _instance(instance)
    M, N, K = 16, 48, 2056
    a = np.ones((M, K), np.float16)
    a[:, 2049:] = 0
    b_kn = np.ones((K, N), np.float16)
    d = np.tile(np.array([1.0, -1.0, -4096.0, 0.5], np.float16), N // 4)[None, :]
    np.testing.assert_array_equal(_run(a, b_kn, [d], [0], ck.Bilinear(1.0, 1.0), instance),
                                  np.broadcast_to(np.tile(np.array([2050, 2048, -2047, 2050], np.float16), N // 4), (M, N)))
    np.testing.assert_array_equal(_run(a, b_kn, [d], [0], ck.Bilinear(2.0, -3.0), instance),
                                  lit.gemm_f16_bilinear(a, b_kn, d, 2.0, -3.0))
    a = uniform_f16((M, 512), -1, 1, 1100)
    b_kn = uniform_f16((512, N), -1, 1, 1101)
    dd = uniform_f16((M, N), -3, 3, 1102)
    np.testing.assert_array_equal(_run(a, b_kn, [dd], [N], ck.Bilinear(0.0, 1.0), instance), dd)
    np.testing.assert_array_equal(_run(a, b_kn, [dd], [N], ck.Bilinear(1.0, 0.0), instance),
                                  gpu_util.gemm_f16(a, np.ascontiguousarray(b_kn.T), instance))


@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 1, "generic"])
def test_fastgelu_limits_through_the_kernel(instance):
    """A = 0: E = fast_gelu(d0 + d1) element by element, including sums far out on both sides (the exponential
    overflows there: the result is x, respectively zero, never NaN)."""
    instance = _instance(instance)
    M, N, K = 32, 64, 64
    a = np.zeros((M, K), np.float16)
    b_kn = uniform_f16((K, N), -1, 1, 1200)
    d0 = np.tile(np.array([0.0, 0.5, -0.5, 3.0, -3.0, 30.0, -30.0, 30000.0], np.float16), N // 8)[None, :]
    d1 = np.tile(np.array([[0.0], [1.0], [-1.0], [-30000.0]], np.float16), (M // 4, N))
    out = _run(a, b_kn, [d0, d1], [0, N], ck.AddAddFastGelu(), instance)
    assert np.isfinite(out).all()
    s = np.broadcast_to(d0, d1.shape).astype(np.float32) + d1.astype(np.float32)
    want = fast.fast_gelu(s).astype(np.float16)
    _close(out, want)
    assert out[0, 0] == 0 and out[0, 7] == np.float16(30000.0) and out[3, 0] == 0


def test_fastgelu_negative_tail_is_pinned():
    """Parity of AddAddFastGelu with the reference's functor is by tolerance, not bit for bit: the device evaluates
    x / (1 + exp(-u)), the reference 0.5 + 0.5 * (2 / (1 + exp(-u)) - 1), whose cancellation makes the factor coarse or
    exactly zero for x below about -5 where the device still returns small negative values. A = 0 turns the GEMM into
    fast_gelu(d0 + d1): a sweep of the sum over [-12, 12] pins the deviation -- at most a few fp16 subnormal steps
    (2^-24 each) in that tail, the suite's rtol = atol = 1e-2 everywhere."""
    M, N, K = 64, 256, 64
    a = np.zeros((M, K), np.float16)
    b_kn = uniform_f16((K, N), -1, 1, 1250)
    s = np.linspace(-12.0, 12.0, M * N, dtype=np.float32).reshape(M, N)
    d0 = np.zeros((1, N), np.float16)
    d1 = s.astype(np.float16)
    out = _run(a, b_kn, [d0, d1], [0, N], ck.AddAddFastGelu(), capi.INSTANCE_AUTO).astype(np.float32)
    x = d1.astype(np.float32)
    want = fast.fast_gelu(x).astype(np.float16).astype(np.float32)
    _close(out.astype(np.float16), want.astype(np.float16))
    tail = x < -5.0
    assert tail.any()
    # in the tail both results are tiny: the device's within 8 fp16 subnormal steps of the reference's, and never positive
    assert np.abs(out[tail] - want[tail]).max() <= 8 * 2.0 ** -24
    assert (out[tail] <= 0).all()


@pytest.mark.parametrize("runs", [2, 3])
def test_k_runs_apply_the_functor_in_the_second_pass(force_k_runs, runs):
    M, N, K = 96, 136, 2048
    a = uniform_f16((M, K), -0.5, 0.5, 1300)
    b_kn = uniform_f16((K, N), -0.5, 0.5, 1301)
    d0, d1 = uniform_f16((1, N), -2, 2, 1302), uniform_f16((M, N), -2, 2, 1303)
    force_k_runs(runs)
    _close(_run(a, b_kn, [d1], [N], ck.Bilinear(0.5, 2.0), workspace=True),
           fast.gemm_f16_bilinear(a, b_kn, d1, 0.5, 2.0))
    _close(_run(a, b_kn, [d0, d1], [0, N], ck.AddAddFastGelu(), instance=2, workspace=True),
           fast.gemm_f16_add_add_fastgelu(a, b_kn, d0, d1))


@pytest.mark.parametrize("layout", list(LAYOUTS))
def test_every_operand_layout_and_ragged_extents(layout):
    """K = 100, N = 50 (no whole 16-byte vectors) and K-major operands go to the element-wise instance."""
    M, N, K = 90, 50, 100
    a = uniform_f16((M, K), -1, 1, 1400)
    b_kn = uniform_f16((K, N), -1, 1, 1401)
    d0, d1 = uniform_f16((1, N), -2, 2, 1402), uniform_f16((M, N), -2, 2, 1403)
    _close(_run(a, b_kn, [d1], [N], ck.Bilinear(1.5, -0.25), layout=layout),
           fast.gemm_f16_bilinear(a, b_kn, d1, 1.5, -0.25))
    _close(_run(a, b_kn, [d0, d1], [0, N], ck.AddAddFastGelu(), layout=layout),
           fast.gemm_f16_add_add_fastgelu(a, b_kn, d0, d1))
    M, N, K = 128, 192, 256
    a = uniform_f16((M, K), -1, 1, 1404)
    b_kn = uniform_f16((K, N), -1, 1, 1405)
    d1 = uniform_f16((M, N), -2, 2, 1406)
    _close(_run(a, b_kn, [d1], [N], ck.Bilinear(1.5, -0.25), layout=layout),
           fast.gemm_f16_bilinear(a, b_kn, d1, 1.5, -0.25))


def test_large_problem_on_the_big_tile():
    """1024 x 1024 x 512 on the 256 x 256 tile: every wave position of the tile epilogue, bias-row and full-tensor D."""
    M, N, K = 1024, 1024, 512
    a = uniform_f16((M, K), -0.5, 0.5, 1500)
    b_kn = uniform_f16((K, N), -0.5, 0.5, 1501)
    d0, d1 = uniform_f16((1, N), -2, 2, 1502), uniform_f16((M, N), -2, 2, 1503)
    _close(_run(a, b_kn, [d1], [N], ck.Bilinear(0.3, 1.7), 0), fast.gemm_f16_bilinear(a, b_kn, d1, 0.3, 1.7))
    _close(_run(a, b_kn, [d0], [0], ck.Bilinear(0.3, 1.7), 0), fast.gemm_f16_bilinear(a, b_kn, d0, 0.3, 1.7))
    _close(_run(a, b_kn, [d0, d1], [0, N], ck.AddAddFastGelu(), 0), fast.gemm_f16_add_add_fastgelu(a, b_kn, d0, d1))
    _close(_run(a, b_kn, [d1, d0], [N, 0], ck.AddAddFastGelu(), 0), fast.gemm_f16_add_add_fastgelu(a, b_kn, d0, d1))


def test_refused_arguments():
    import ctypes as C
    L = capi.lib()
    q = L.ckx_gemm_f16_multiple_d_is_supported
    assert q(64, 64, 64, 64, 64, 64, 0, 64, 0, 1, 0, capi.EPI_BILINEAR, -1) == capi.OK
    assert q(64, 64, 64, 64, 64, 0, 64, 64, 0, 1, 0, capi.EPI_ADD_ADD_FASTGELU, -1) == capi.OK
    assert q(64, 64, 64, 64, 64, 8, 0, 64, 0, 1, 0, capi.EPI_BILINEAR, -1) == capi.UNSUPPORTED          # D stride < N
    assert q(64, 64, 64, 64, 64, 0, 8, 64, 0, 1, 0, capi.EPI_ADD_ADD_FASTGELU, -1) == capi.UNSUPPORTED
    # the bilinear operation carries scalars: it has its own entry point
    assert L.ckx_gemm_f16_multiple_d(1, 1, 1, 1, 1, 64, 64, 64, 64, 64, 64, 0, 64, 0, 1, 0, capi.EPI_BILINEAR, -1, None, 0,
                                     None) == capi.INVALID_VALUE
    # null D pointers
    assert L.ckx_gemm_f16_bilinear(1, 1, None, 1, 64, 64, 64, 64, 64, 64, 64, 0, 1, 0, C.c_float(1), C.c_float(1), -1, None,
                                   0, None) == capi.INVALID_VALUE
    assert L.ckx_gemm_f16_multiple_d(1, 1, 1, None, 1, 64, 64, 64, 64, 64, 0, 64, 64, 0, 1, 0, capi.EPI_ADD_ADD_FASTGELU, -1,
                                     None, 0, None) == capi.INVALID_VALUE
    # not for the int8 family, the batched operators or the conv operators
    assert L.ckx_gemm_i8_is_supported(64, 64, 64, 64, 64, 64, 0, 1, 0, capi.EPI_BILINEAR, -1) == capi.UNSUPPORTED
    d = capi.Conv2dDesc(1, 8, 8, 4, 4, 1, 1, 4, 4, 1, 1, 1, 1, 0, 0, 0, 0)
    assert L.ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(d), capi.EPI_ADD_ADD_FASTGELU, -1) != capi.OK
    with pytest.raises(ValueError):
        ck.DeviceGemmMultipleDF16().MakeArgumentPointer(1, 1, [1], 1, 8, 8, 8, 8, 8, [8], 8, None, None, ck.AddAddFastGelu())
    with pytest.raises(ValueError):
        ck.DeviceGemmMultipleDF16().MakeArgumentPointer(1, 1, [1, 1], 1, 8, 8, 8, 8, 8, [8, 8], 8, None, None,
                                                        ck.Bilinear(1, 1))
