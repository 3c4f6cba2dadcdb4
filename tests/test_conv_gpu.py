"""GPU parity: NHWC implicit-GEMM conv2d forward through the C ABI against the CPU oracle.

Parameter sets follow the reference's test/convnd_fwd/conv2d_fwd.cpp:104-115,187-266
(default 3x3 stride 2 dilation 2 pad 2; 1x1 stride 1 pad 0; 1x1 stride 2 pad 0) and its golden
vectors (test/reference_conv_fwd/reference_conv_fwd.cpp:94-154), plus benchmark configuration 4's
ResNet-50 layers on a reduced batch (full batch through the im2col/BLAS form).
int8 is bit-exact (PassThrough keeps the low byte, as the reference's int8 conv does);
fp16 within rtol = atol = 1e-2.
"""
import json
import os

import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8
from oracle import fast, lit

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
RTOL = ATOL = 1e-2

# (N, C, K, Hi, Wi, Y, X, strides, dilations, pads)
SMALL = [
    (2, 16, 32, 9, 11, 3, 3, (2, 2), (2, 2), (2, 2)),     # reference "default" shape family
    (2, 32, 48, 8, 8, 1, 1, (1, 1), (1, 1), (0, 0)),      # Filter1x1Stride1Pad0
    (2, 32, 16, 9, 9, 1, 1, (2, 2), (1, 1), (0, 0)),      # Filter1x1Pad0
    (3, 16, 80, 7, 5, 3, 2, (1, 2), (1, 1), (1, 0)),      # asymmetric everything
    (1, 64, 64, 14, 14, 3, 3, (1, 1), (1, 1), (1, 1)),
    (4, 48, 24, 6, 6, 5, 5, (1, 1), (1, 1), (2, 2)),      # C not a multiple of the K tile
]


def _f16_close(out, ref):
    bad, max_err = lit.check_err_f16(out, ref, RTOL, ATOL)
    assert bad == 0, f"{bad} outside tolerance, max err {max_err}"


@pytest.mark.parametrize("case", SMALL)
@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 0, 2, 4, 6, 7, 8])
def test_conv2d_int8_small_cases_bit_exact(case, instance):
    import gpu_util
    N, C, K, Hi, Wi, Y, X, s, d, p = case
    inp = uniform_int8((N, Hi, Wi, C), -5, 5, 100 + C)
    wei = uniform_int8((K, Y, X, C), -5, 5, 200 + K)
    out = gpu_util.conv2d_fwd(inp, wei, s, d, p, instance=instance)
    np.testing.assert_array_equal(out, lit.conv2d_fwd(inp, wei, s, d, p))
    rq = ck.RequantReluRequant(0.05, 0.7, rounded=True)
    out = gpu_util.conv2d_fwd(inp, wei, s, d, p, out_op=rq, instance=instance)
    np.testing.assert_array_equal(
        out, lit.conv2d_fwd(inp, wei, s, d, p, epi=lit.EPI_REQUANT_RND, scale_gemm=0.05, scale_relu=0.7))


@pytest.mark.parametrize("case", SMALL)
@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 1, 3, 5, 8])
def test_conv2d_fp16_small_cases(case, instance):
    import gpu_util
    N, C, K, Hi, Wi, Y, X, s, d, p = case
    inp = uniform_f16((N, Hi, Wi, C), -1, 1, 300 + C)
    wei = uniform_f16((K, Y, X, C), -1, 1, 400 + K)
    out = gpu_util.conv2d_fwd(inp, wei, s, d, p, instance=instance)
    _f16_close(out, lit.conv2d_fwd(inp, wei, s, d, p))


def test_conv2d_reference_golden_vectors_fp16():
    """The reference's own expected outputs. They are fp32 there; the fp16 operator adds exactly
    one round-to-nearest-even of the (exact) fp32 sum, e.g. 1138.5 -> 1138."""
    import gpu_util
    gold = json.load(open(os.path.join(HERE, "golden", "reference_conv_fwd_vectors.json")))
    for case in gold["cases"]:
        N, K, C = case["N"], case["K"], case["C"]
        Hi, Wi = case["input"]
        Y, X = case["filter"]
        # C = 2 as in the reference case (4-byte pixels: the element-wise instance), and the same two channels
        # embedded in 8 (zeros elsewhere leave every sum unchanged: the vectorised instances)
        want = np.array(case["expected"], np.float32).astype(np.float16)
        for cpad in (C, 8):
            inp = np.zeros((N, Hi, Wi, cpad), np.float16)
            inp[..., :C] = np.arange(N * Hi * Wi * C, dtype=np.float32).reshape(N, Hi, Wi, C)
            wei = np.zeros((K, Y, X, cpad), np.float16)
            wei[..., :C] = 0.5
            out = gpu_util.conv2d_fwd(inp, wei, case["strides"], case["dilations"], case["left_pads"],
                                      right_pads=case["right_pads"])
            np.testing.assert_array_equal(out.ravel(), want)


RESNET = [
    # benchmark configuration 4 (C, K, filter, HW, stride, pad)
    (64, 64, 3, 56, 1, 1),
    (256, 512, 1, 56, 2, 0),
    (512, 512, 3, 7, 1, 1),
]


@pytest.mark.parametrize("layer", RESNET)
@pytest.mark.parametrize("dtype", ["int8", "fp16"])
def test_conv2d_config4_resnet50_layers(layer, dtype):
    """Full N=256 launch; every image is checked against the im2col/BLAS form, two images
    against the literal ReferenceConvFwd restatement."""
    import gpu_util
    C, K, f, HW, st, pd = layer
    N = 256
    s, d, p = (st, st), (1, 1), (pd, pd)
    if dtype == "int8":
        inp = uniform_int8((N, HW, HW, C), -5, 5, 500 + C)
        wei = uniform_int8((K, f, f, C), -5, 5, 600 + K)
        rq = ck.RequantReluRequant(0.01, 0.5, rounded=True)
        out = gpu_util.conv2d_fwd(inp, wei, s, d, p, out_op=rq)
        for n0 in range(0, N, 32):
            np.testing.assert_array_equal(
                out[n0:n0 + 32],
                fast.conv2d_fwd_i8(inp[n0:n0 + 32], wei, s, d, p, epi=lit.EPI_REQUANT_RND, scale_gemm=0.01,
                                   scale_relu=0.5))
        for n in (0, N - 1):
            np.testing.assert_array_equal(
                out[n:n + 1], lit.conv2d_fwd(inp[n:n + 1], wei, s, d, p, epi=lit.EPI_REQUANT_RND,
                                             scale_gemm=0.01, scale_relu=0.5))
        # PassThrough: low byte of the sum
        out = gpu_util.conv2d_fwd(inp[:8], wei, s, d, p)
        np.testing.assert_array_equal(out, fast.conv2d_fwd_i8(inp[:8], wei, s, d, p))
    else:
        inp = uniform_f16((N, HW, HW, C), -1, 1, 700 + C)
        wei = uniform_f16((K, f, f, C), -1, 1, 800 + K)
        out = gpu_util.conv2d_fwd(inp, wei, s, d, p)
        for n0 in range(0, N, 32):
            _f16_close(out[n0:n0 + 32], fast.conv2d_fwd_f16(inp[n0:n0 + 32], wei, s, d, p))
        _f16_close(out[:1], lit.conv2d_fwd(inp[:1], wei, s, d, p))


@pytest.mark.parametrize("layer", RESNET)
def test_conv2d_fp16_resnet50_layers_integer_operands_bit_exact(layer):
    """Integers in [-3, 3] (the reference profiler's integer initialisation, narrowed so that the largest sum,
    9 * 9 * 512, stays inside fp16): fp32 accumulation is exact in any order, so the fp16 output of the input-patch,
    pointwise and tile kernels must equal the rounded exact sums bit for bit -- no tolerance to hide a wrong tap,
    channel or pixel behind. Full N = 256 launch, every image checked."""
    import gpu_util
    C, K, f, HW, st, pd = layer
    N = 256
    s, d, p = (st, st), (1, 1), (pd, pd)
    inp = uniform_int8((N, HW, HW, C), -3, 3, 510 + C).astype(np.float16)
    wei = uniform_int8((K, f, f, C), -3, 3, 610 + K).astype(np.float16)
    out = gpu_util.conv2d_fwd(inp, wei, s, d, p)
    for n0 in range(0, N, 32):
        # (the BLAS form is exact here too: integers below 2^24 in fp32)
        np.testing.assert_array_equal(out[n0:n0 + 32], fast.conv2d_fwd_f16(inp[n0:n0 + 32], wei, s, d, p))


def test_conv2d_unsupported_arguments_are_refused():
    import torch
    d = torch.zeros(1 << 16, dtype=torch.int8, device="cuda")
    op = ck.DeviceConv2dFwdInt8()
    # C = 3 (the reference's OddC case) is not a whole 16-byte vector: the vectorised instances refuse it
    fast_op = ck.DeviceConv2dFwdInt8(0)
    arg = fast_op.MakeArgumentPointer(d, d, d, 1, 8, 3, [8, 8], [3, 3], [6, 6], [1, 1], [1, 1], [0, 0], [0, 0])
    assert not fast_op.IsSupportedArgument(arg)
    with pytest.raises(RuntimeError):
        fast_op.MakeInvokerPointer().Run(arg)
    assert op.IsSupportedArgument(op.MakeArgumentPointer(d, d, d, 1, 8, 3, [8, 8], [3, 3], [6, 6], [1, 1], [1, 1], [0, 0], [0, 0]))
    # output size inconsistent with the geometry
    arg = op.MakeArgumentPointer(d, d, d, 1, 8, 16, [8, 8], [3, 3], [7, 6], [1, 1], [1, 1], [0, 0], [0, 0])
    assert not op.IsSupportedArgument(arg)


# (N, Hi, Wi, pads): fp16, C = K = 64, 3x3, stride 1, dilation 1, Wo = 56 -- the input-patch kernel's shapes
PATCH = [
    (2, 9, 56, (1, 1)),       # partial last band (Ho = 9)
    (1, 4, 56, (1, 1)),       # a single band
    (3, 12, 58, (1, 0)),      # no horizontal padding
    (2, 7, 54, (0, 2)),       # wide horizontal padding, none vertically (Ho = 5)
    (1, 56, 56, (1, 1)),      # the ResNet-50 conv2_x layer, one image
]


@pytest.mark.parametrize("case", PATCH)
@pytest.mark.parametrize("auto", [True, False])
def test_conv2d_fp16_input_patch_kernel(case, auto):
    """The LDS-resident input-patch kernel (explicit instance and automatic choice) against the
    literal oracle; the tile kernel must agree on the same problem."""
    import gpu_util
    N, Hi, Wi, p = case
    inp = uniform_f16((N, Hi, Wi, 64), -1, 1, 900 + Hi)
    wei = uniform_f16((64, 3, 3, 64), -1, 1, 901 + Wi)
    patch = gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Patch")
    out = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), p, instance=capi.INSTANCE_AUTO if auto else patch)
    ref = lit.conv2d_fwd(inp, wei, (1, 1), (1, 1), p)
    assert out.shape == ref.shape and out.shape[2] == 56
    _f16_close(out, ref)
    _f16_close(gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), p, instance=7), ref)


def test_conv2d_fp16_input_patch_kernel_more_images_than_cus():
    """Workgroups walk several images: 300 images on at most 256 workgroups."""
    import gpu_util
    inp = uniform_f16((300, 5, 56, 64), -1, 1, 77)
    wei = uniform_f16((64, 3, 3, 64), -0.5, 0.5, 78)
    out = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), (1, 1))
    _f16_close(out, fast.conv2d_fwd_f16(inp, wei, (1, 1), (1, 1), (1, 1)))


def test_conv2d_input_patch_instance_refuses_other_shapes():
    import ctypes as C
    import gpu_util
    patch = gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Patch")
    d = capi.Conv2dDesc(2, 64, 64, 9, 48, 3, 3, 9, 48, 1, 1, 1, 1, 1, 1, 1, 1)     # Wo = 48
    assert capi.lib().ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(d), 0, patch) == capi.UNSUPPORTED
    assert capi.lib().ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(d), 0, -1) == capi.OK
    assert capi.lib().ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_I8, C.byref(d), 0, patch) == capi.UNSUPPORTED
    n = capi.lib().ckx_num_instances(capi.OP_CONV2D_FWD_I8)
    assert capi.lib().ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_I8, C.byref(d), 0, n) == capi.INVALID_VALUE


@pytest.mark.parametrize("case", PATCH)
@pytest.mark.parametrize("auto", [True, False])
def test_conv2d_int8_input_patch_kernel_bit_exact(case, auto):
    """The int8 form of the input-patch kernel (a pixel = 64 bytes = one MFMA k-step): PassThrough (low byte)
    and both requant epilogues, bit for bit against the literal oracle; the tile kernel must agree."""
    import gpu_util
    N, Hi, Wi, p = case
    inp = uniform_int8((N, Hi, Wi, 64), -5, 5, 950 + Hi)
    wei = uniform_int8((64, 3, 3, 64), -5, 5, 951 + Wi)
    patch = gpu_util.conv_instance(capi.OP_CONV2D_FWD_I8, "Patch")
    inst = capi.INSTANCE_AUTO if auto else patch
    out = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), p, instance=inst)
    ref = lit.conv2d_fwd(inp, wei, (1, 1), (1, 1), p)
    assert out.shape == ref.shape and out.shape[2] == 56
    np.testing.assert_array_equal(out, ref)
    for rq, kind in ((ck.RequantReluRequant(0.05, 0.7, rounded=True), lit.EPI_REQUANT_RND),
                     (ck.RequantReluRequant(0.03, 1.0), lit.EPI_REQUANT_CK)):
        out = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), p, out_op=rq, instance=inst)
        ref = lit.conv2d_fwd(inp, wei, (1, 1), (1, 1), p, epi=kind, scale_gemm=rq.scale_gemm, scale_relu=rq.scale_relu)
        np.testing.assert_array_equal(out, ref)
        np.testing.assert_array_equal(gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), p, out_op=rq, instance=7), ref)
        assert out.max() > 0


def test_conv2d_int8_input_patch_kernel_full_range_and_many_images():
    """Full-range int8 values (the int32 sums wrap into the low byte under PassThrough) and more images than
    workgroups."""
    import gpu_util
    inp = uniform_int8((300, 5, 56, 64), -128, 127, 87)
    wei = uniform_int8((64, 3, 3, 64), -128, 127, 88)
    out = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), (1, 1))
    np.testing.assert_array_equal(out, fast.conv2d_fwd_i8(inp, wei, (1, 1), (1, 1), (1, 1)))


# (N, Hi, Wi, pads): C = K = 128, 3x3, stride 1, dilation 1, Wo = 28 -- the second shape of the input-patch instance
# (ResNet-50 conv3_x: eight waves that share the pixels, weights in registers)
PATCH_WIDE = [
    (2, 9, 28, (1, 1)),       # partial last band (Ho = 9)
    (1, 4, 28, (1, 1)),       # a single band
    (3, 12, 30, (1, 0)),      # no horizontal padding
    (2, 7, 26, (0, 2)),       # wide horizontal padding, none vertically (Ho = 5)
    (1, 28, 28, (1, 1)),      # the ResNet-50 conv3_x layer, one image (seven bands: the ring wraps, its first rows are loaded twice)
    (2, 70, 28, (1, 1)),      # eighteen bands: every ring position several times
]


@pytest.mark.parametrize("case", PATCH_WIDE)
def test_conv2d_fp16_input_patch_kernel_128_channels(case):
    """The 128-channel form of the input-patch instance against the literal oracle (sampled images for the tall case);
    the tile kernel must agree on the same problem."""
    import gpu_util
    N, Hi, Wi, p = case
    inp = uniform_f16((N, Hi, Wi, 128), -1, 1, 700 + Hi)
    wei = uniform_f16((128, 3, 3, 128), -1, 1, 701 + Wi)
    patch = gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Patch")
    out = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), p, instance=patch)
    ref = fast.conv2d_fwd_f16(inp, wei, (1, 1), (1, 1), p) if Hi > 30 else lit.conv2d_fwd(inp, wei, (1, 1), (1, 1), p)
    assert out.shape == ref.shape and out.shape[2] == 28
    _f16_close(out, ref)
    _f16_close(gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), p, instance=7), ref)


@pytest.mark.parametrize("case", PATCH_WIDE)
def test_conv2d_int8_input_patch_kernel_128_channels_bit_exact(case):
    """... int8: PassThrough (low byte) and both requant epilogues, bit for bit."""
    import gpu_util
    N, Hi, Wi, p = case
    inp = uniform_int8((N, Hi, Wi, 128), -5, 5, 750 + Hi)
    wei = uniform_int8((128, 3, 3, 128), -5, 5, 751 + Wi)
    patch = gpu_util.conv_instance(capi.OP_CONV2D_FWD_I8, "Patch")
    out = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), p, instance=patch)
    np.testing.assert_array_equal(out, fast.conv2d_fwd_i8(inp, wei, (1, 1), (1, 1), p))
    for rq, kind in ((ck.RequantReluRequant(0.02, 0.7, rounded=True), lit.EPI_REQUANT_RND),
                     (ck.RequantReluRequant(0.015, 1.0), lit.EPI_REQUANT_CK)):
        out = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), p, out_op=rq, instance=patch)
        ref = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), p, out_op=rq, instance=7)
        np.testing.assert_array_equal(out, ref)
        if Hi <= 12:
            np.testing.assert_array_equal(out, lit.conv2d_fwd(inp, wei, (1, 1), (1, 1), p, epi=kind, scale_gemm=rq.scale_gemm,
                                                              scale_relu=rq.scale_relu))
        assert out.max() > 0


def test_conv2d_input_patch_kernel_128_channels_many_images_and_automatic_choice():
    """More images than workgroups, through the automatic choice (which takes the instance from 112 images on); integer
    fp16 operands make the fp32 sums exact, so the result must equal the rounded exact product."""
    import gpu_util
    inp = uniform_int8((300, 5, 28, 128), -3, 3, 97)
    wei = uniform_int8((128, 3, 3, 128), -3, 3, 98)
    d = capi.Conv2dDesc(300, 128, 128, 5, 28, 3, 3, 5, 28, 1, 1, 1, 1, 1, 1, 1, 1)
    patch = gpu_util.conv_instance(capi.OP_CONV2D_FWD_I8, "Patch")
    assert capi.conv2d_fwd_plan(capi.OP_CONV2D_FWD_I8, d, capi.EPI_PASSTHROUGH, 0)[0] == patch
    np.testing.assert_array_equal(gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), (1, 1)),
                                  fast.conv2d_fwd_i8(inp, wei, (1, 1), (1, 1), (1, 1)))
    out = gpu_util.conv2d_fwd(inp.astype(np.float16), wei.astype(np.float16), (1, 1), (1, 1), (1, 1))
    exact = fast.conv2d_fwd_f16(inp.astype(np.float16), wei.astype(np.float16), (1, 1), (1, 1), (1, 1))
    np.testing.assert_array_equal(out, exact)


# (N, C, K, Hi, Wi, strides): 1x1 filters, no padding, a pixel of 256 or 512 bytes, K in blocks of 512 -- the
# weight-stationary pointwise kernel's shapes (the reference's Filter1x1Pad0 / Filter1x1Stride1Pad0 specialisations)
POINTWISE_F16 = [
    (1, 256, 512, 4, 8, (1, 1)),        # one band exactly
    (3, 256, 512, 7, 5, (1, 1)),        # pixel count not a multiple of the band (105)
    (2, 128, 1024, 9, 9, (2, 2)),       # 256-byte pixels, two blocks of output channels, stride 2
    (2, 256, 512, 11, 13, (2, 1)),      # different strides along h and w
    (1, 128, 512, 1, 3, (1, 1)),        # fewer pixels than one MFMA tile
]
POINTWISE_I8 = [
    (1, 256, 512, 4, 8, (1, 1)),
    (3, 512, 512, 7, 5, (1, 1)),        # 512-byte pixels
    (2, 256, 1024, 9, 9, (2, 2)),
    (2, 512, 512, 11, 13, (1, 2)),
]


@pytest.mark.parametrize("case", POINTWISE_F16)
def test_conv2d_fp16_pointwise_kernel(case):
    """The weight-stationary 1x1 kernel (weights in registers, pixels through an LDS ring) against the literal
    oracle; the tile kernel must agree on the same problem."""
    import gpu_util
    N, C, K, Hi, Wi, s = case
    inp = uniform_f16((N, Hi, Wi, C), -1, 1, 1000 + Hi)
    wei = uniform_f16((K, 1, 1, C), -1, 1, 1001 + Wi)
    pw = gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Pointwise")
    ref = lit.conv2d_fwd(inp, wei, s, (1, 1), (0, 0))
    _f16_close(gpu_util.conv2d_fwd(inp, wei, s, (1, 1), (0, 0), instance=pw), ref)
    _f16_close(gpu_util.conv2d_fwd(inp, wei, s, (1, 1), (0, 0), instance=0), ref)


@pytest.mark.parametrize("case", POINTWISE_I8)
def test_conv2d_int8_pointwise_kernel_bit_exact(case):
    import gpu_util
    N, C, K, Hi, Wi, s = case
    inp = uniform_int8((N, Hi, Wi, C), -5, 5, 1010 + Hi)
    wei = uniform_int8((K, 1, 1, C), -5, 5, 1011 + Wi)
    pw = gpu_util.conv_instance(capi.OP_CONV2D_FWD_I8, "Pointwise")
    np.testing.assert_array_equal(gpu_util.conv2d_fwd(inp, wei, s, (1, 1), (0, 0), instance=pw),
                                  lit.conv2d_fwd(inp, wei, s, (1, 1), (0, 0)))
    for rq, kind in ((ck.RequantReluRequant(0.02, 0.7, rounded=True), lit.EPI_REQUANT_RND),
                     (ck.RequantReluRequant(0.03, 1.0), lit.EPI_REQUANT_CK)):
        out = gpu_util.conv2d_fwd(inp, wei, s, (1, 1), (0, 0), out_op=rq, instance=pw)
        np.testing.assert_array_equal(
            out, lit.conv2d_fwd(inp, wei, s, (1, 1), (0, 0), epi=kind, scale_gemm=rq.scale_gemm, scale_relu=rq.scale_relu))
        assert out.max() > 0


@pytest.mark.parametrize("dtype", ["f16", "i8"])
def test_conv2d_pointwise_kernel_long_runs_of_bands(dtype):
    """Enough pixels for every workgroup to go round its ring of bands several times (the automatic choice for such
    layers), full-range int8 values included (the int32 sums wrap into the low byte under PassThrough)."""
    import gpu_util
    if dtype == "f16":
        inp = uniform_f16((36, 56, 56, 256), -1, 1, 1020)
        wei = uniform_f16((512, 1, 1, 256), -1, 1, 1021)
        out = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), (0, 0))
        _f16_close(out, fast.conv2d_fwd_f16(inp, wei, (1, 1), (1, 1), (0, 0)))
    else:
        inp = uniform_int8((256, 57, 55, 256), -128, 127, 1022)
        wei = uniform_int8((512, 1, 1, 256), -128, 127, 1023)
        out = gpu_util.conv2d_fwd(inp, wei, (2, 2), (1, 1), (0, 0))
        np.testing.assert_array_equal(out, fast.conv2d_fwd_i8(inp, wei, (2, 2), (1, 1), (0, 0)))


def test_conv2d_pointwise_instance_refuses_other_shapes():
    import ctypes as C
    import gpu_util
    L = capi.lib()
    pw = gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Pointwise")
    ok = capi.Conv2dDesc(2, 512, 256, 8, 8, 1, 1, 8, 8, 1, 1, 1, 1, 0, 0, 0, 0)
    assert L.ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(ok), 0, pw) == capi.OK
    for d in (capi.Conv2dDesc(2, 256, 256, 8, 8, 1, 1, 8, 8, 1, 1, 1, 1, 0, 0, 0, 0),      # K = 256
              capi.Conv2dDesc(2, 512, 64, 8, 8, 1, 1, 8, 8, 1, 1, 1, 1, 0, 0, 0, 0),       # 128-byte pixels
              capi.Conv2dDesc(2, 512, 256, 8, 8, 1, 1, 10, 10, 1, 1, 1, 1, 1, 1, 1, 1),    # padded
              capi.Conv2dDesc(2, 512, 256, 8, 8, 3, 3, 6, 6, 1, 1, 1, 1, 0, 0, 0, 0)):     # 3x3
        assert L.ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(d), 0, pw) == capi.UNSUPPORTED
        assert L.ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(d), 0, -1) == capi.OK
    # the residual functor stays with the tile kernel
    assert L.ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(ok), capi.EPI_ADD_RELU_ADD, pw) == capi.UNSUPPORTED


# (N, C, K, Hi, Wi): 1x1, stride 1, no padding
ROWS_F16 = [
    (1, 32, 64, 3, 5),          # 64-byte pixels, 15 rows: less than one tile of 16
    (3, 32, 128, 7, 5),         # 105 rows: a ragged last tile and a ragged last pair of tiles
    (2, 64, 256, 9, 11),        # 128-byte pixels (ResNet conv2_x: 64 -> 256)
    (2, 64, 64, 8, 8),
    (2, 32, 192, 5, 6),         # three of the four 64-column groups of a block
    (1, 64, 512, 6, 7),         # two blocks of 256 output channels
    (2, 128, 128, 7, 9),        # 256-byte pixels (up to 128 output channels)
    (2, 256, 64, 9, 7),         # 512-byte pixels (64 output channels: ResNet conv2_x, 256 -> 64), one row tile per iteration
]
ROWS_I8 = [
    (1, 64, 64, 3, 5),          # 64-byte pixels
    (3, 64, 256, 7, 5),
    (2, 128, 512, 9, 11),       # 128-byte pixels, two blocks of output channels (ResNet conv3_x: 128 -> 512)
    (2, 128, 128, 8, 8),
    (2, 64, 768, 5, 5),         # three blocks
    (2, 256, 128, 7, 9),        # 256-byte pixels
    (3, 512, 64, 5, 7),         # 512-byte pixels
]


@pytest.mark.parametrize("case", ROWS_F16)
def test_conv2d_fp16_streaming_1x1_kernel(case):
    """The streaming 1x1 kernel (weights in registers, pixel rows straight into MFMA operands, no LDS) against the
    literal oracle; the tile kernel must agree on the same problem."""
    import gpu_util
    N, C, K, Hi, Wi = case
    inp = uniform_f16((N, Hi, Wi, C), -1, 1, 1100 + Hi)
    wei = uniform_f16((K, 1, 1, C), -1, 1, 1101 + Wi)
    rows = gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Rows<")
    ref = lit.conv2d_fwd(inp, wei, (1, 1), (1, 1), (0, 0))
    _f16_close(gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), (0, 0), instance=rows), ref)
    _f16_close(gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), (0, 0), instance=3), ref)


@pytest.mark.parametrize("case", ROWS_I8)
def test_conv2d_int8_streaming_1x1_kernel_bit_exact(case):
    import gpu_util
    N, C, K, Hi, Wi = case
    inp = uniform_int8((N, Hi, Wi, C), -5, 5, 1110 + Hi)
    wei = uniform_int8((K, 1, 1, C), -5, 5, 1111 + Wi)
    rows = gpu_util.conv_instance(capi.OP_CONV2D_FWD_I8, "Rows<")
    np.testing.assert_array_equal(gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), (0, 0), instance=rows),
                                  lit.conv2d_fwd(inp, wei, (1, 1), (1, 1), (0, 0)))
    for rq, kind in ((ck.RequantReluRequant(0.02, 0.7, rounded=True), lit.EPI_REQUANT_RND),
                     (ck.RequantReluRequant(0.03, 1.0), lit.EPI_REQUANT_CK)):
        out = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), (0, 0), out_op=rq, instance=rows)
        np.testing.assert_array_equal(
            out, lit.conv2d_fwd(inp, wei, (1, 1), (1, 1), (0, 0), epi=kind, scale_gemm=rq.scale_gemm, scale_relu=rq.scale_relu))
        assert out.max() > 0


@pytest.mark.parametrize("dtype", ["f16", "i8"])
def test_conv2d_streaming_1x1_kernel_every_wave_several_rounds(dtype):
    """ResNet conv2_x at a batch that gives every wave of the full launch several pairs of row tiles (the automatic
    choice for such layers), full-range int8 values included."""
    import gpu_util
    if dtype == "f16":
        inp = uniform_f16((48, 56, 56, 64), -1, 1, 1120)
        wei = uniform_f16((64, 1, 1, 64), -1, 1, 1121)
        desc = capi.Conv2dDesc(48, 64, 64, 56, 56, 1, 1, 56, 56, 1, 1, 1, 1, 0, 0, 0, 0)
        assert capi.conv2d_fwd_plan(capi.OP_CONV2D_FWD_F16, desc)[0] == gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Rows<")
        out = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), (0, 0))
        _f16_close(out, fast.conv2d_fwd_f16(inp, wei, (1, 1), (1, 1), (0, 0)))
    else:
        inp = uniform_int8((96, 56, 56, 64), -128, 127, 1122)
        wei = uniform_int8((64, 1, 1, 64), -128, 127, 1123)
        desc = capi.Conv2dDesc(96, 64, 64, 56, 56, 1, 1, 56, 56, 1, 1, 1, 1, 0, 0, 0, 0)
        assert capi.conv2d_fwd_plan(capi.OP_CONV2D_FWD_I8, desc)[0] == gpu_util.conv_instance(capi.OP_CONV2D_FWD_I8, "Rows<")
        out = gpu_util.conv2d_fwd(inp, wei, (1, 1), (1, 1), (0, 0))
        np.testing.assert_array_equal(out, fast.conv2d_fwd_i8(inp, wei, (1, 1), (1, 1), (0, 0)))


def test_conv2d_streaming_1x1_instance_refuses_other_shapes():
    import ctypes as C
    import gpu_util
    L = capi.lib()
    rows = gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Rows<")
    ok = capi.Conv2dDesc(2, 256, 64, 8, 8, 1, 1, 8, 8, 1, 1, 1, 1, 0, 0, 0, 0)
    assert L.ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(ok), 0, rows) == capi.OK
    for d in (capi.Conv2dDesc(2, 96, 64, 8, 8, 1, 1, 8, 8, 1, 1, 1, 1, 0, 0, 0, 0),        # K = 96: not whole 64-column groups
              capi.Conv2dDesc(2, 320, 64, 8, 8, 1, 1, 8, 8, 1, 1, 1, 1, 0, 0, 0, 0),       # K = 320: above 256, not whole blocks
              capi.Conv2dDesc(2, 256, 128, 8, 8, 1, 1, 8, 8, 1, 1, 1, 1, 0, 0, 0, 0),      # 256-byte pixels with 256 output channels
              capi.Conv2dDesc(2, 128, 256, 8, 8, 1, 1, 8, 8, 1, 1, 1, 1, 0, 0, 0, 0),      # 512-byte pixels with 128
              capi.Conv2dDesc(2, 64, 512, 8, 8, 1, 1, 8, 8, 1, 1, 1, 1, 0, 0, 0, 0),       # 1024-byte pixels
              capi.Conv2dDesc(2, 256, 64, 8, 8, 1, 1, 4, 4, 2, 2, 1, 1, 0, 0, 0, 0),       # stride 2
              capi.Conv2dDesc(2, 256, 64, 8, 8, 1, 1, 10, 10, 1, 1, 1, 1, 1, 1, 1, 1),     # padded
              capi.Conv2dDesc(2, 256, 64, 8, 8, 3, 3, 6, 6, 1, 1, 1, 1, 0, 0, 0, 0)):      # 3x3
        assert L.ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(d), 0, rows) == capi.UNSUPPORTED
        assert L.ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(d), 0, -1) == capi.OK
    # the residual functor and the per-channel scales stay with the tile kernel
    assert L.ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(ok), capi.EPI_ADD_RELU_ADD, rows) == capi.UNSUPPORTED
    assert L.ckx_conv2d_fwd_is_supported(capi.OP_CONV2D_FWD_I8, C.byref(ok), capi.EPI_MUL2_CLAMP, rows) == capi.UNSUPPORTED


@pytest.mark.parametrize("shape", ["patch", "pointwise"])
def test_conv2d_specialists_fall_back_on_unaligned_output(shape):
    """The input-patch and pointwise kernels store whole 16-byte vectors: an output that starts 2 bytes into a buffer
    is not theirs. The automatic choice must run such a problem on a tile instance (element stores), the explicit
    instance must refuse it."""
    import torch
    import gpu_util
    if shape == "patch":
        inp, wei, s, p = uniform_f16((2, 8, 56, 64), -1, 1, 1030), uniform_f16((64, 3, 3, 64), -1, 1, 1031), (1, 1), (1, 1)
    else:
        inp, wei, s, p = uniform_f16((40, 56, 56, 256), -1, 1, 1032), uniform_f16((512, 1, 1, 256), -1, 1, 1033), (2, 2), (0, 0)
    N, Hi, Wi, Cc = inp.shape
    K, Y, X, _ = wei.shape
    Ho, Wo = (Hi + 2 * p[0] - Y) // s[0] + 1, (Wi + 2 * p[1] - X) // s[1] + 1
    di, dw = gpu_util.dev(inp), gpu_util.dev(wei)
    buf = torch.full((N * Ho * Wo * K + 8,), float("nan"), dtype=torch.float16, device="cuda")
    out = buf[1:1 + N * Ho * Wo * K]
    geom = (N, K, Cc, [Hi, Wi], [Y, X], [Ho, Wo], list(s), [1, 1], list(p), list(p), None, None, None)
    op = ck.DeviceConv2dFwdF16()
    arg = op.MakeArgumentPointer(di, dw, out.data_ptr(), *geom)
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    host = buf.cpu().numpy()
    assert np.isnan(host[0]) and np.isnan(host[1 + N * Ho * Wo * K:]).all()
    _f16_close(host[1:1 + N * Ho * Wo * K].reshape(N, Ho, Wo, K), fast.conv2d_fwd_f16(inp, wei, s, (1, 1), p))
    special = ck.DeviceConv2dFwdF16(gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Patch" if shape == "patch" else "Pointwise"))
    arg = special.MakeArgumentPointer(di, dw, out.data_ptr(), *geom)
    with pytest.raises(RuntimeError):
        special.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
