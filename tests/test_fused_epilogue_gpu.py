"""GPU parity of the fused bias / ReLU / residual epilogues of the fp16 operators, through the C ABI:

  * conv2d forward + bias + ReLU (+ residual add): DeviceConvFwdBiasActivation[Add]
    (examples 06 / 07; host references reference_conv_fwd_bias_activation[_add].hpp)
  * GEMM + D tensors: DeviceGemmMultipleD with AddRelu on the fp16-rounded C (example 03) and
    AddReluAdd in fp32

against the CPU oracle, rtol = atol = 1e-2 (the fp16 bar), plus cases chosen so that the
result is exact and a wrong order of operations shows.
"""
import json
import os

import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_f16
from oracle import fast, lit

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
RTOL = ATOL = 1e-2

with open(os.path.join(HERE, "golden", "reference_conv_fwd_vectors.json")) as f:
    GOLD = json.load(f)

# (N, C, K, Hi, Wi, Y, X, strides, dilations, pads)
CONV = [
    (2, 16, 32, 9, 11, 3, 3, (2, 2), (2, 2), (2, 2)),
    (2, 32, 48, 8, 8, 1, 1, (1, 1), (1, 1), (0, 0)),
    (3, 16, 80, 7, 5, 3, 2, (1, 2), (1, 1), (1, 0)),
    (1, 64, 64, 14, 14, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 8, 20, 6, 6, 3, 3, (1, 1), (1, 1), (1, 1)),       # K not a multiple of 8: unaligned D rows
]


def _close(out, ref):
    bad, max_err = lit.check_err_f16(out, ref, RTOL, ATOL)
    assert bad == 0, f"{bad} outside tolerance, max err {max_err}"


def _conv(inp, wei, bias, resi, s, d, p, instance=capi.INSTANCE_AUTO, workspace=False):
    import torch
    import gpu_util
    N, Hi, Wi, C = inp.shape
    K, Y, X, _ = wei.shape
    Ho = (Hi + 2 * p[0] - ((Y - 1) * d[0] + 1)) // s[0] + 1
    Wo = (Wi + 2 * p[1] - ((X - 1) * d[1] + 1)) // s[1] + 1
    di, dw, db = gpu_util.dev(inp), gpu_util.dev(wei), gpu_util.dev(bias)
    do = torch.full((N, Ho, Wo, K), float("nan"), dtype=torch.float16, device="cuda")
    op = ck.DeviceConv2dFwdBiasActivationF16(instance)
    geom = (N, K, C, [Hi, Wi], [Y, X], [Ho, Wo], list(s), list(d), list(p), list(p), None, None)
    if resi is None:
        arg = op.MakeArgumentPointer(di, dw, do, db, *geom, ck.AddRelu())
    else:
        dr = gpu_util.dev(resi)
        arg = op.MakeArgumentPointer(di, dw, do, db, dr, *geom, ck.AddReluAdd())
    assert op.IsSupportedArgument(arg), capi.last_error()
    if workspace:
        need = op.GetWorkSpaceSize(arg)
        ws = torch.full((max(need, 16),), 0x7F, dtype=torch.uint8, device="cuda")
        op.SetWorkSpacePointer(arg, ws)
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    return do.cpu().numpy()


@pytest.mark.parametrize("case", CONV)
@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 0, 1, 3, 6, 7, 8])
def test_conv2d_bias_relu_and_residual(case, instance):
    N, C, K, Hi, Wi, Y, X, s, d, p = case
    inp = uniform_f16((N, Hi, Wi, C), -1, 1, 300 + C)
    wei = uniform_f16((K, Y, X, C), -1, 1, 400 + K)
    bias = uniform_f16((K,), -2, 2, 500 + K)
    ref = lit.conv2d_fwd_bias_relu_f16(inp, wei, bias, None, s, d, p)
    out = _conv(inp, wei, bias, None, s, d, p, instance)
    _close(out, ref)
    assert (out == 0).any() and (out > 0).any()          # the ReLU is in play
    resi = uniform_f16(ref.shape, -2, 2, 600 + K)
    _close(_conv(inp, wei, bias, resi, s, d, p, instance), lit.conv2d_fwd_bias_relu_f16(inp, wei, bias, resi, s, d, p))


@pytest.mark.parametrize("case", [c for c in GOLD["cases"] if max(c["expected"]) < 2000 and
                                  c["left_pads"] == c["right_pads"]])
def test_conv2d_bias_relu_golden_vectors_exact(case):
    """The reference's golden conv outputs pushed through the functors by hand (exact in fp16):
    relu(acc + b) + r with a negative r differs from relu(acc + b + r). The golden cases have 2
    input channels; they are padded with zero channels to the 16-byte vector the kernels need."""
    N, K, C = case["N"], case["K"], case["C"]
    Hi, Wi = case["input"]
    Y, X = case["filter"]
    inp = np.zeros((N, Hi, Wi, 8), np.float16)
    inp[..., :C] = np.arange(N * Hi * Wi * C, dtype=np.float32).reshape(N, Hi, Wi, C)
    wei = np.full((K, Y, X, 8), 0.5, np.float16)
    n, k, ho, wo = case["out_dims_nkhw"]
    gold = np.array(case["expected"], np.float32).reshape(n, ho, wo, k)
    bias = (-np.median(gold) - 0.5 * np.arange(K)).astype(np.float16)
    resi = np.full(gold.shape, -3.0, np.float16)
    want = np.maximum(gold + bias.astype(np.float32), 0)
    args = (case["strides"], case["dilations"], case["left_pads"])
    np.testing.assert_array_equal(_conv(inp, wei, bias, None, *args), want.astype(np.float16))
    np.testing.assert_array_equal(_conv(inp, wei, bias, resi, *args), (want - 3.0).astype(np.float16))


def test_conv2d_bias_relu_resnet_layer_and_split_k(force_k_runs):
    """ResNet-50 3x3 layer on a reduced batch against the im2col/BLAS form, also with the K loop
    cut into runs (the second pass applies the functor)."""
    inp = uniform_f16((4, 14, 14, 256), -1, 1, 31)
    wei = uniform_f16((256, 3, 3, 256), -0.2, 0.2, 32)
    bias = uniform_f16((256,), -3, 3, 33)
    resi = uniform_f16((4, 14, 14, 256), -2, 2, 34)
    ref = fast.conv2d_fwd_bias_relu_f16(inp, wei, bias, resi, (1, 1), (1, 1), (1, 1))
    _close(_conv(inp, wei, bias, resi, (1, 1), (1, 1), (1, 1)), ref)
    force_k_runs(3)
    _close(_conv(inp, wei, bias, resi, (1, 1), (1, 1), (1, 1), workspace=True), ref)
    _close(_conv(inp, wei, bias, None, (1, 1), (1, 1), (1, 1), instance=2, workspace=True),
           fast.conv2d_fwd_bias_relu_f16(inp, wei, bias, None, (1, 1), (1, 1), (1, 1)))


@pytest.mark.parametrize("instance", [1, 7])
@pytest.mark.parametrize("filt", [1, 3])
def test_conv2d_bias_relu_several_tiles_per_workgroup(instance, filt):
    """The 256 x 128 and 256 x 64 instances on 588 row tiles: more than the persistent grid has workgroups, so most
    of them finish a tile, hand the zeroed accumulators back to the K loop and finish another (these two instances
    issue their matrix instructions outside the compiler's view and order that hand-over themselves). 3x3 with
    padding and 1x1, bias + ReLU and the residual form."""
    C, K, pad = (32, 128, 1) if filt == 3 else (64, 128, 0)
    inp = uniform_f16((48, 56, 56, C), -1, 1, 71)
    wei = uniform_f16((K, filt, filt, C), -0.3, 0.3, 72)
    bias = uniform_f16((K,), -3, 3, 73)
    resi = uniform_f16((48, 56, 56, K), -2, 2, 74)
    args = ((1, 1), (1, 1), (pad, pad))
    _close(_conv(inp, wei, bias, None, *args, instance=instance), fast.conv2d_fwd_bias_relu_f16(inp, wei, bias, None, *args))
    _close(_conv(inp, wei, bias, resi, *args, instance=instance), fast.conv2d_fwd_bias_relu_f16(inp, wei, bias, resi, *args))


def _gemm_md(a, b_nk, ds, strides, op_functor, instance=capi.INSTANCE_AUTO, lde=None):
    import torch
    import gpu_util
    M, K = a.shape
    N = b_nk.shape[0]
    lde = lde or N
    da, db = gpu_util.dev(a), gpu_util.dev(b_nk)
    dds = [gpu_util.dev(d) for d in ds]
    de = torch.full((M, lde), float("nan"), dtype=torch.float16, device="cuda")
    op = ck.DeviceGemmMultipleDF16(instance)
    arg = op.MakeArgumentPointer(da, db, dds, de, M, N, K, K, K, strides, lde, None, None, op_functor)
    if not op.IsSupportedArgument(arg):
        return None
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    return de.cpu().numpy()[:, :N]


@pytest.mark.parametrize("shape", [(256, 256, 256), (300, 200, 128), (17, 130, 1040), (5, 48, 4096), (64, 100, 80),
                                   (513, 88, 512)])
@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 0, 2, 5, 9, 11, 13])
def test_gemm_bias_relu_like_example_03(shape, instance):
    """E = AddRelu(half(A*B), D) with D a bias row (stride 0, as example 03 passes it) and a full
    [M,N] tensor; every instance family incl. the skinny ones."""
    M, N, K = shape
    a = uniform_f16((M, K), -1, 1, 700 + M)
    b_nk = uniform_f16((N, K), -1, 1, 701 + N)
    bias = uniform_f16((1, N), -3, 3, 702 + N)
    out = _gemm_md(a, b_nk, [bias], [0], ck.AddRelu(), instance)
    if out is None:
        assert instance >= 9     # a skinny instance with fewer rows than M
        return
    _close(out, lit.gemm_f16_add_relu(a, b_nk.T, bias))
    assert (out == 0).any() and (out > 0).any()
    d_full = uniform_f16((M, N), -3, 3, 703 + N)
    _close(_gemm_md(a, b_nk, [d_full], [N], ck.AddRelu(), instance), lit.gemm_f16_add_relu(a, b_nk.T, d_full))


def test_gemm_add_relu_rounds_c_first_exact():
    """K = 2049 ones: acc = 2049 -> fp16 2048; + 1 -> 2049 -> 2048 (ties to even). One rounding of
    2050 would store 2050."""
    a = np.ones((48, 2056), np.float16)
    a[:, 2049:] = 0
    b_nk = np.ones((40, 2056), np.float16)
    d = np.tile(np.array([1.0, -1.0, -4096.0, 0.0], np.float16), 10)[None, :]
    out = _gemm_md(a, b_nk, [d], [0], ck.AddRelu())
    np.testing.assert_array_equal(out, np.broadcast_to(np.tile(np.array([2048, 2047, 0, 2048], np.float16), 10), (48, 40)))
    assert not np.signbit(out).any()


@pytest.mark.parametrize("shape", [(256, 256, 256), (130, 72, 1040), (9, 48, 512)])
def test_gemm_add_relu_add_fp32_functor(shape):
    """AddReluAdd as a CDE operation: relu(acc + D0) + D1 in fp32, one rounding; D0 a bias row, D1 a
    residual tensor with a padded row stride; E with a padded row stride as well."""
    M, N, K = shape
    a = uniform_f16((M, K), -1, 1, 800 + M)
    b_nk = uniform_f16((N, K), -1, 1, 801 + N)
    bias = uniform_f16((1, N), -3, 3, 802)
    resi_padded = uniform_f16((M, N + 8), -2, 2, 803)
    out = _gemm_md(a, b_nk, [bias, resi_padded], [0, N + 8], ck.AddReluAdd(), lde=N + 16)
    acc = a.astype(np.float32) @ b_nk.T.astype(np.float32)
    ref = (np.maximum(acc + bias.astype(np.float32), 0) + resi_padded[:, :N].astype(np.float32)).astype(np.float16)
    _close(out, ref)


def test_fused_epilogue_argument_checks():
    L = capi.lib()
    ok = L.ckx_gemm_f16_multiple_d_is_supported(64, 64, 64, 64, 64, 0, 0, 64, 0, 1, 0, capi.EPI_CSHUFFLE_ADD_RELU, -1)
    assert ok == capi.OK
    assert L.ckx_gemm_f16_multiple_d_is_supported(64, 64, 64, 64, 64, 8, 0, 64, 0, 1, 0, capi.EPI_ADD_RELU, -1) == capi.UNSUPPORTED
    assert L.ckx_gemm_f16_multiple_d_is_supported(64, 64, 64, 64, 64, 0, 0, 64, 0, 1, 0, capi.EPI_REQUANT_CK, -1) == capi.INVALID_VALUE
    assert L.ckx_gemm_i8_is_supported(64, 64, 64, 64, 64, 64, 0, 1, 0, capi.EPI_ADD_RELU, -1) == capi.UNSUPPORTED
    d = capi.Conv2dDesc(1, 8, 8, 4, 4, 1, 1, 4, 4, 1, 1, 1, 1, 0, 0, 0, 0)
    import ctypes as C
    assert L.ckx_conv2d_fwd_bias_activation_f16(1, 1, 1, 0, 0, C.byref(d), capi.EPI_ADD_RELU, -1, 0, 0, None) == capi.INVALID_VALUE
    assert L.ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_I8, C.byref(d), capi.EPI_ADD_RELU, -1) != capi.OK


@pytest.mark.parametrize("shape", [(2, 9, 56, (1, 1)), (1, 56, 56, (1, 1)), (3, 6, 58, (0, 0))])
@pytest.mark.parametrize("auto", [True, False])
def test_conv2d_bias_relu_on_the_input_patch_kernel(shape, auto):
    """ResNet conv2_x shapes (C = K = 64, 3x3, Wo = 56) take the input-patch kernel, fused functors included."""
    N, Hi, Wi, p = shape
    inp = uniform_f16((N, Hi, Wi, 64), -1, 1, 950 + Hi)
    wei = uniform_f16((64, 3, 3, 64), -0.5, 0.5, 951)
    bias = uniform_f16((64,), -2, 2, 952)
    import gpu_util
    inst = capi.INSTANCE_AUTO if auto else gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Patch")
    ref = lit.conv2d_fwd_bias_relu_f16(inp, wei, bias, None, (1, 1), (1, 1), p)
    out = _conv(inp, wei, bias, None, (1, 1), (1, 1), p, inst)
    _close(out, ref)
    assert (out == 0).any() and (out > 0).any()
    resi = uniform_f16(ref.shape, -2, 2, 953)
    _close(_conv(inp, wei, bias, resi, (1, 1), (1, 1), p, inst),
           lit.conv2d_fwd_bias_relu_f16(inp, wei, bias, resi, (1, 1), (1, 1), p))


@pytest.mark.parametrize("shape", [(2, 9, 28, (1, 1)), (1, 28, 28, (1, 1)), (3, 6, 30, (0, 0))])
def test_conv2d_bias_relu_on_the_input_patch_kernel_128_channels(shape):
    """ResNet conv3_x shapes (C = K = 128, 3x3, Wo = 28) on the input-patch instance with bias + ReLU compiled in; the
    residual form is not one of its epilogues (explicit instance refused, the automatic choice takes a tile instance)."""
    N, Hi, Wi, p = shape
    inp = uniform_f16((N, Hi, Wi, 128), -1, 1, 960 + Hi)
    wei = uniform_f16((128, 3, 3, 128), -0.5, 0.5, 961)
    bias = uniform_f16((128,), -2, 2, 962)
    import gpu_util
    inst = gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Patch")
    ref = lit.conv2d_fwd_bias_relu_f16(inp, wei, bias, None, (1, 1), (1, 1), p)
    out = _conv(inp, wei, bias, None, (1, 1), (1, 1), p, inst)
    _close(out, ref)
    assert (out == 0).any() and (out > 0).any()
    resi = uniform_f16(ref.shape, -2, 2, 963)
    with pytest.raises(AssertionError):
        _conv(inp, wei, bias, resi, (1, 1), (1, 1), p, inst)
    _close(_conv(inp, wei, bias, resi, (1, 1), (1, 1), p, capi.INSTANCE_AUTO),
           lit.conv2d_fwd_bias_relu_f16(inp, wei, bias, resi, (1, 1), (1, 1), p))


@pytest.mark.parametrize("shape", [(3, 32, 64, 7, 5), (2, 64, 256, 9, 11), (2, 32, 192, 5, 6), (1, 64, 512, 6, 7), (24, 64, 64, 56, 56)])
def test_conv2d_bias_relu_on_the_streaming_1x1_kernel(shape):
    """1x1 stride-1 layers with pixels of 64 / 128 bytes on the streaming kernel with the bias + ReLU functor compiled in
    (explicit instance for the small shapes, the automatic choice for the ResNet conv2_x one); the residual form is not
    one of its epilogues."""
    import gpu_util
    N, C, K, Hi, Wi = shape
    inp = uniform_f16((N, Hi, Wi, C), -1, 1, 81)
    wei = uniform_f16((K, 1, 1, C), -0.5, 0.5, 82)
    bias = uniform_f16((K,), -3, 3, 83)
    big = N * Hi * Wi >= 65536
    inst = capi.INSTANCE_AUTO if big else gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Rows<")
    ref = (fast if big else lit).conv2d_fwd_bias_relu_f16(inp, wei, bias, None, (1, 1), (1, 1), (0, 0))
    _close(_conv(inp, wei, bias, None, (1, 1), (1, 1), (0, 0), instance=inst), ref)
    if not big:
        resi = uniform_f16((N, Hi, Wi, K), -2, 2, 84)
        with pytest.raises(AssertionError):
            _conv(inp, wei, bias, resi, (1, 1), (1, 1), (0, 0), instance=inst)


@pytest.mark.parametrize("shape", [(3, 256, 512, 7, 5, (1, 1)), (2, 128, 1024, 9, 9, (2, 2)), (40, 256, 512, 56, 56, (2, 2))])
def test_conv2d_bias_relu_on_the_pointwise_kernel(shape):
    """1x1 layers on the weight-stationary kernel with the bias + ReLU functor compiled in (explicit instance for the
    small shapes, the automatic choice for the large one)."""
    import gpu_util
    N, C, K, Hi, Wi, s = shape
    inp = uniform_f16((N, Hi, Wi, C), -1, 1, 960 + Hi)
    wei = uniform_f16((K, 1, 1, C), -0.5, 0.5, 961)
    bias = uniform_f16((K,), -2, 2, 962)
    big = N * Hi * Wi > 100000
    inst = capi.INSTANCE_AUTO if big else gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Pointwise")
    ref = (fast if big else lit).conv2d_fwd_bias_relu_f16(inp, wei, bias, None, s, (1, 1), (0, 0))
    out = _conv(inp, wei, bias, None, s, (1, 1), (0, 0), inst)
    _close(out, ref)
    assert (out == 0).any() and (out > 0).any()
