"""GPU parity: int8 GEMM and conv2d with ONE REQUANT SCALE PER OUTPUT COLUMN / CHANNEL (the D operand) through the
C ABI against the CPU oracle, bit for bit.

The functor is upstream Composable Kernel's Activation_Mul2_Clamp<PassThrough / Relu>
(ck/tensor_operation/gpu/element/quantization_operation.hpp as shipped with ROCm) behind the reference's
DeviceGemmMultipleD interface (device_gemm_multiple_d.hpp:14-55); the reference snapshot has no instance of it, so
there are no reference vectors: the oracle's restatement is pinned in tests/test_oracle.py (against the reference's
RequantReluRequant, which the Relu form equals at scaleGemm = 1, against exact dyadic arithmetic and brute force),
and the same identities are checked on the GPU here. Every instance of the int8 GEMM family takes the functor
(tile, skinny, element-wise), with and without a K split, and so do the conv specialists (patch-window kernel;
pointwise kernel for 256-byte pixels); batches do not.
"""
import ctypes as C

import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_int8
from oracle import fast, lit

pytestmark = pytest.mark.gpu

N_INSTANCES = 19
SKINNY_MAX_M = {9: 16, 10: 32, 11: 64, 12: 16, 13: 16, 14: 16, 15: 32, 16: 32, 17: 128}
ACTS = {"relu": ck.Relu, "passthrough": ck.PassThrough}


def scales_for(n, seed):
    """per-column scales of both signs, with zeros, tiny values and values that saturate"""
    rng = np.random.default_rng(seed)
    s = rng.uniform(-0.05, 0.05, n).astype(np.float32)
    s[::7] = 0.0
    s[3::11] = rng.uniform(5.0, 50.0, len(s[3::11])).astype(np.float32)      # clamps at 127 / -128
    s[5::13] = np.float32(2.0 ** -20)
    return s


def run_gemm(a, b_nk, scales, act, instance=capi.INSTANCE_AUTO, lde=None, layouts=(ck.RowMajor, ck.ColumnMajor),
             workspace=False, allow_unsupported=False):
    import torch
    import gpu_util
    al, bl = layouts
    M, K = a.shape
    N = b_nk.shape[0]
    lde = lde or N
    a_dev = gpu_util.dev(a if al is ck.RowMajor else np.ascontiguousarray(a.T))
    b_dev = gpu_util.dev(b_nk if bl is ck.ColumnMajor else np.ascontiguousarray(b_nk.T))
    sa = K if al is ck.RowMajor else M
    sb = K if bl is ck.ColumnMajor else N
    d_dev = gpu_util.dev(scales)
    e_dev = torch.full((M, lde), 77, dtype=torch.int8, device="cuda")
    op = ck.DeviceGemmMultipleDInt8(instance, ALayout=al, BLayout=bl)
    arg = op.MakeArgumentPointer(a_dev, b_dev, [d_dev], e_dev, M, N, K, sa, sb, [0], lde, ck.PassThrough(),
                                 ck.PassThrough(), ck.ActivationMul2Clamp(ACTS[act]()))
    if allow_unsupported and not op.IsSupportedArgument(arg):
        return None
    assert op.IsSupportedArgument(arg), capi.last_error()
    ws = None
    if workspace:
        need = op.GetWorkSpaceSize(arg)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        op.SetWorkSpacePointer(arg, ws, need)
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream(), False))
    torch.cuda.synchronize()
    out = e_dev.cpu().numpy()
    assert np.all(out[:, N:] == 77), "wrote outside the E rows"
    return out[:, :N]


@pytest.mark.parametrize("act", list(ACTS))
@pytest.mark.parametrize("instance", range(N_INSTANCES))
@pytest.mark.parametrize("shape", [(256, 256, 256), (300, 200, 128), (17, 130, 1040), (1, 64, 16), (64, 16, 80),
                                   (513, 80, 2048)])
def test_every_instance_bit_exact(instance, shape, act):
    M, N, K = shape
    a = uniform_int8((M, K), -8, 8, 21 + M)
    b_nk = uniform_int8((N, K), -8, 8, 23 + N)
    s = scales_for(N, 5 + N)
    out = run_gemm(a, b_nk, s, act, instance=instance, lde=N + 16, allow_unsupported=True)
    if out is None:
        assert instance in SKINNY_MAX_M and M > SKINNY_MAX_M[instance]
        return
    want = fast.gemm_i8_mul2_clamp(a, b_nk.T, s, act == "relu")
    np.testing.assert_array_equal(out, want)
    assert len(np.unique(want)) > 3


def test_literal_oracle_small():
    a = uniform_int8((40, 96), -20, 20, 1)
    b_nk = uniform_int8((24, 96), -20, 20, 2)
    s = scales_for(24, 3)
    for act in ACTS:
        np.testing.assert_array_equal(run_gemm(a, b_nk, s, act), lit.gemm_i8_mul2_clamp(a, b_nk.T, s, act == "relu"))


@pytest.mark.parametrize("runs", [2, 3, 5])
@pytest.mark.parametrize("shape", [(128, 512, 4096), (64, 200, 8192), (300, 130, 2048)])
def test_k_runs_through_the_workspace(shape, runs, force_k_runs):
    """the second pass of a K split applies the per-column functor: bit-identical to the single pass"""
    M, N, K = shape
    a = uniform_int8((M, K), -8, 8, 31)
    b_nk = uniform_int8((N, K), -8, 8, 32)
    s = scales_for(N, 33)
    want = fast.gemm_i8_mul2_clamp(a, b_nk.T, s, True)
    force_k_runs(runs)
    nk = K // 128
    expect = runs if -(-nk // runs) * (runs - 1) < nk else 1     # every run needs at least one K tile
    for instance in (0, 2, 4):
        assert capi.gemm_plan(capi.OP_GEMM_I8, M, N, K, epilogue=capi.EPI_RELU_MUL2_CLAMP, workspace_bytes=1 << 30,
                              instance=instance)[1] == expect
        np.testing.assert_array_equal(run_gemm(a, b_nk, s, "relu", instance=instance, workspace=True), want)


@pytest.mark.parametrize("layouts", [(ck.ColumnMajor, ck.ColumnMajor), (ck.RowMajor, ck.RowMajor),
                                     (ck.ColumnMajor, ck.RowMajor)])
def test_k_major_operands(layouts):
    a = uniform_int8((272, 384), -8, 8, 41)
    b_nk = uniform_int8((208, 384), -8, 8, 42)
    s = scales_for(208, 43)
    for act in ACTS:
        np.testing.assert_array_equal(run_gemm(a, b_nk, s, act, layouts=layouts),
                                      fast.gemm_i8_mul2_clamp(a, b_nk.T, s, act == "relu"))


def test_padding_shapes_take_the_element_wise_instance():
    """K = 100 and an odd N: the element-granular instance, chosen by AUTO"""
    a = uniform_int8((70, 100), -8, 8, 51)
    b_nk = uniform_int8((45, 100), -8, 8, 52)
    s = scales_for(45, 53)
    np.testing.assert_array_equal(run_gemm(a, b_nk, s, "relu"), fast.gemm_i8_mul2_clamp(a, b_nk.T, s, True))


def test_equal_scales_reproduce_the_reference_functor():
    """Relu form with one scale s in every column == the reference's RequantReluRequant(1, s), literal form
    (example 14): both are trunc(clamp(s * relu(float(acc)))). GPU against GPU and against the oracle."""
    import gpu_util
    a = uniform_int8((192, 320), -8, 8, 61)
    b_nk = uniform_int8((144, 320), -8, 8, 62)
    for s in (0.03, 0.4, 1.0, 2.5):
        per_col = run_gemm(a, b_nk, np.full(144, s, np.float32), "relu")
        per_tensor = gpu_util.gemm_i8(a, b_nk, ck.RequantReluRequant(1.0, s))
        np.testing.assert_array_equal(per_col, per_tensor)
        np.testing.assert_array_equal(per_col, lit.gemm_i8(a, b_nk.T, lit.EPI_REQUANT_CK, 1.0, s))


def test_columns_are_independent():
    """column n of the per-column result == column n of a run with scale[n] everywhere"""
    a = uniform_int8((96, 256), -8, 8, 71)
    b_nk = uniform_int8((80, 256), -8, 8, 72)
    s = scales_for(80, 73)
    out = run_gemm(a, b_nk, s, "passthrough")
    for n in (0, 3, 7, 31, 79):
        one = run_gemm(a, b_nk, np.full(80, s[n], np.float32), "passthrough")
        np.testing.assert_array_equal(out[:, n], one[:, n])


def _conv(x, w, s, act, strides, pads, instance=capi.INSTANCE_AUTO, allow_unsupported=False):
    import torch
    import gpu_util
    N, Hi, Wi, C_ = x.shape
    K, Y, X, _ = w.shape
    Ho = lit.conv_out_len(Hi, Y, strides[0], 1, pads[0], pads[0])
    Wo = lit.conv_out_len(Wi, X, strides[1], 1, pads[1], pads[1])
    dx, dw, ds = gpu_util.dev(x), gpu_util.dev(w), gpu_util.dev(s)
    dy = torch.full((N, Ho, Wo, K), 77, dtype=torch.int8, device="cuda")
    op = ck.DeviceConv2dFwdMultipleDInt8(instance)
    arg = op.MakeArgumentPointer(dx, dw, dy, ds, N, K, C_, [Hi, Wi], [Y, X], [Ho, Wo], list(strides), [1, 1], list(pads),
                                 list(pads), ck.PassThrough(), ck.PassThrough(), ck.ActivationMul2Clamp(ACTS[act]()))
    if allow_unsupported and not op.IsSupportedArgument(arg):
        return None
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream(), False))
    torch.cuda.synchronize()
    return dy.cpu().numpy()


@pytest.mark.parametrize("layer", [(2, 64, 64, 3, 56, 1, 1), (3, 256, 512, 1, 28, 2, 0), (4, 32, 48, 3, 17, 2, 1),
                                   (2, 3, 24, 3, 20, 1, 1)])
def test_conv2d_per_output_channel(layer):
    """N, C, K, filter, HW, stride, pad: the patch-window and pointwise shapes (which fall back to the tile instances
    for this functor), a ragged layer, and the reference's C = 3 case on the element-wise instance"""
    n, c, k, f, hw, st, pd = layer
    x = uniform_int8((n, hw, hw, c), -5, 5, 81)
    w = uniform_int8((k, f, f, c), -5, 5, 82)
    s = scales_for(k, 83)
    for act in ACTS:
        out = _conv(x, w, s, act, (st, st), (pd, pd))
        np.testing.assert_array_equal(out, fast.conv2d_fwd_i8_mul2_clamp(x, w, s, act == "relu", (st, st), (1, 1), (pd, pd)))


@pytest.mark.parametrize("act", list(ACTS))
def test_conv_specialists_take_the_functor(act):
    """the patch-window kernel (3x3, C = K = 64, Wo = 56) and the pointwise kernel (1x1, 256-byte pixels) with one
    scale per output channel, forced and as the automatic choice; 512-byte pixels stay on the tile instances"""
    import gpu_util
    patch = gpu_util.conv_instance(capi.OP_CONV2D_FWD_I8, "Patch")
    point = gpu_util.conv_instance(capi.OP_CONV2D_FWD_I8, "Pointwise")
    relu = act == "relu"
    x = uniform_int8((5, 56, 56, 64), -5, 5, 91)
    w = uniform_int8((64, 3, 3, 64), -5, 5, 92)
    s = scales_for(64, 93)
    want = fast.conv2d_fwd_i8_mul2_clamp(x, w, s, relu, (1, 1), (1, 1), (1, 1))
    np.testing.assert_array_equal(_conv(x, w, s, act, (1, 1), (1, 1), instance=patch), want)
    x = uniform_int8((3, 28, 28, 256), -5, 5, 94)
    w = uniform_int8((512, 1, 1, 256), -5, 5, 95)
    s = scales_for(512, 96)
    want = fast.conv2d_fwd_i8_mul2_clamp(x, w, s, relu, (2, 2), (1, 1), (0, 0))
    np.testing.assert_array_equal(_conv(x, w, s, act, (2, 2), (0, 0), instance=point), want)
    x = uniform_int8((2, 14, 14, 512), -5, 5, 97)
    w = uniform_int8((512, 1, 1, 512), -5, 5, 98)
    assert _conv(x, w, s, act, (1, 1), (0, 0), instance=point, allow_unsupported=True) is None
    np.testing.assert_array_equal(_conv(x, w, s, act, (1, 1), (0, 0)),
                                  fast.conv2d_fwd_i8_mul2_clamp(x, w, s, relu, (1, 1), (1, 1), (0, 0)))


def test_conv_automatic_choice_reaches_the_specialists():
    """batches large enough for the planner to prefer them (N >= 112 for the patch kernel, 16 K pixels for pointwise)"""
    x = uniform_int8((112, 56, 56, 64), -5, 5, 101)
    w = uniform_int8((64, 3, 3, 64), -5, 5, 102)
    s = scales_for(64, 103)
    d = capi.Conv2dDesc(112, 64, 64, 56, 56, 3, 3, 56, 56, 1, 1, 1, 1, 1, 1, 1, 1)
    import gpu_util
    assert capi.conv2d_fwd_plan(capi.OP_CONV2D_FWD_I8, d, capi.EPI_RELU_MUL2_CLAMP, 0)[0] == \
        gpu_util.conv_instance(capi.OP_CONV2D_FWD_I8, "Patch")
    np.testing.assert_array_equal(_conv(x, w, s, "relu", (1, 1), (1, 1)),
                                  fast.conv2d_fwd_i8_mul2_clamp(x, w, s, True, (1, 1), (1, 1), (1, 1)))
    x = uniform_int8((32, 56, 56, 256), -5, 5, 104)
    w = uniform_int8((512, 1, 1, 256), -5, 5, 105)
    s = scales_for(512, 106)
    d = capi.Conv2dDesc(32, 512, 256, 56, 56, 1, 1, 28, 28, 2, 2, 1, 1, 0, 0, 0, 0)
    assert capi.conv2d_fwd_plan(capi.OP_CONV2D_FWD_I8, d, capi.EPI_MUL2_CLAMP, 0)[0] == \
        gpu_util.conv_instance(capi.OP_CONV2D_FWD_I8, "Pointwise")
    np.testing.assert_array_equal(_conv(x, w, s, "passthrough", (2, 2), (0, 0)),
                                  fast.conv2d_fwd_i8_mul2_clamp(x, w, s, False, (2, 2), (1, 1), (0, 0)))


def test_refused_arguments():
    L = capi.lib()
    q = L.ckx_gemm_i8_multiple_d_is_supported
    assert q(64, 64, 64, 64, 64, 0, 64, 0, 1, 0, capi.EPI_RELU_MUL2_CLAMP, -1) == capi.OK
    assert q(64, 64, 64, 64, 64, 64, 64, 0, 1, 0, capi.EPI_RELU_MUL2_CLAMP, -1) == capi.UNSUPPORTED   # a [M, N] scale tensor
    assert q(64, 64, 64, 64, 64, 0, 64, 0, 1, 0, capi.EPI_REQUANT_RND, -1) == capi.INVALID_VALUE
    assert q(64, 64, 64, 64, 64, 0, 64, 0, 1, 0, capi.EPI_ADD_RELU, -1) == capi.INVALID_VALUE
    # the plain entry points have no D operand to take the scales from
    assert L.ckx_gemm_i8_is_supported(64, 64, 64, 64, 64, 64, 0, 1, 0, capi.EPI_MUL2_CLAMP, -1) == capi.UNSUPPORTED
    assert L.ckx_gemm_f16_multiple_d_is_supported(64, 64, 64, 64, 64, 0, 0, 64, 0, 1, 0, capi.EPI_MUL2_CLAMP, -1) \
        == capi.INVALID_VALUE
    import torch
    a = torch.zeros((64, 64), dtype=torch.int8, device="cuda")
    e = torch.zeros((64, 64), dtype=torch.int8, device="cuda")
    st = L.ckx_gemm_i8_multiple_d(a.data_ptr(), a.data_ptr(), None, e.data_ptr(), 64, 64, 64, 64, 64, 0, 64, 0, 1, 0,
                                  capi.EPI_MUL2_CLAMP, -1, None, 0, None)
    assert st == capi.INVALID_VALUE and b"null D operand" in L.ckx_last_error()
    st = L.ckx_gemm_i8(a.data_ptr(), a.data_ptr(), e.data_ptr(), 64, 64, 64, 64, 64, 64, 0, 1, 0, capi.EPI_MUL2_CLAMP,
                       C.c_float(1), C.c_float(1), -1, None, 0, None)
    assert st == capi.INVALID_VALUE
