"""The stem conv instance (conv_stem.hpp): C = 3, 7 x 7, stride 2, padding 3, K = 64 -- the first layer of the
reference's ResNet-50 script (script/profile_resnet50.sh:46), which its own instance lists reach through the OddC
specialisation. Through the C ABI against the CPU oracle (ReferenceConvFwd restated, oracle/ck_oracle.cpp): int8
bit-exact with every requant form, fp16 within rtol = atol = 1e-2 and bit-exact on integer operands, the fused
bias + ReLU form against the reference's conv + AddRelu; image sizes whose output rows and columns are not whole bands
and tiles; the automatic choice and the element-granular instance on the same inputs."""
import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8
from oracle import lit

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2
S, D, P = (2, 2), (1, 1), (3, 3)
# (N, Hi, Wi): whole tiles and bands (224 -> 112 = 7 x 16, 28 x 4), one tile, ragged columns / rows / both, tiny
SIZES = [(2, 224, 224), (3, 32, 32), (2, 30, 50), (1, 17, 9), (2, 64, 40), (1, 7, 7), (5, 2, 66)]


def _stem(op):
    import gpu_util
    return gpu_util.conv_instance(op, "Stem")


def _f16_close(out, ref):
    bad, max_err = lit.check_err_f16(out, ref, RTOL, ATOL)
    assert bad == 0, f"{bad} outside tolerance, max err {max_err}"


@pytest.mark.parametrize("size", SIZES)
@pytest.mark.parametrize("auto", [False, True])
def test_stem_int8_bit_exact(size, auto):
    import gpu_util
    N, Hi, Wi = size
    inp = uniform_int8((N, Hi, Wi, 3), -5, 5, 7000 + Hi)
    wei = uniform_int8((64, 7, 7, 3), -5, 5, 7001 + Wi)
    inst = capi.INSTANCE_AUTO if auto else _stem(capi.OP_CONV2D_FWD_I8)
    if auto:
        Ho, Wo = (Hi + 6 - 7) // 2 + 1, (Wi + 6 - 7) // 2 + 1
        d = capi.Conv2dDesc(N, 64, 3, Hi, Wi, 7, 7, Ho, Wo, 2, 2, 1, 1, 3, 3, 3, 3)
        assert capi.conv2d_fwd_plan(capi.OP_CONV2D_FWD_I8, d)[0] == _stem(capi.OP_CONV2D_FWD_I8)
    np.testing.assert_array_equal(gpu_util.conv2d_fwd(inp, wei, S, D, P, instance=inst), lit.conv2d_fwd(inp, wei, S, D, P))
    for rounded, epi in ((True, lit.EPI_REQUANT_RND), (False, lit.EPI_REQUANT_CK)):
        rq = ck.RequantReluRequant(0.01, 0.5, rounded=rounded)
        np.testing.assert_array_equal(gpu_util.conv2d_fwd(inp, wei, S, D, P, out_op=rq, instance=inst),
                                      lit.conv2d_fwd(inp, wei, S, D, P, epi=epi, scale_gemm=0.01, scale_relu=0.5))


@pytest.mark.parametrize("size", SIZES)
def test_stem_fp16(size):
    import gpu_util
    N, Hi, Wi = size
    inst = _stem(capi.OP_CONV2D_FWD_F16)
    inp = uniform_f16((N, Hi, Wi, 3), -1, 1, 7100 + Hi)
    wei = uniform_f16((64, 7, 7, 3), -1, 1, 7101 + Wi)
    _f16_close(gpu_util.conv2d_fwd(inp, wei, S, D, P, instance=inst), lit.conv2d_fwd(inp, wei, S, D, P))
    # integer operands: every partial sum is an integer below 2^24, the result is exact in any order
    inp = uniform_int8((N, Hi, Wi, 3), -5, 5, 7102).astype(np.float16)
    wei = uniform_int8((64, 7, 7, 3), -5, 5, 7103).astype(np.float16)
    np.testing.assert_array_equal(gpu_util.conv2d_fwd(inp, wei, S, D, P, instance=inst), lit.conv2d_fwd(inp, wei, S, D, P))
    # ... and the element-granular instance (the reference's OddC route) agrees on the same inputs
    generic = gpu_util.conv_instance(capi.OP_CONV2D_FWD_F16, "Generic")
    np.testing.assert_array_equal(gpu_util.conv2d_fwd(inp, wei, S, D, P, instance=inst),
                                  gpu_util.conv2d_fwd(inp, wei, S, D, P, instance=generic))


@pytest.mark.parametrize("size", SIZES[:4])
@pytest.mark.parametrize("auto", [False, True])
def test_stem_fp16_bias_relu(size, auto):
    from test_fused_epilogue_gpu import _conv
    N, Hi, Wi = size
    inp = uniform_f16((N, Hi, Wi, 3), -1, 1, 7200 + Hi)
    wei = uniform_f16((64, 7, 7, 3), -1, 1, 7201 + Wi)
    bias = uniform_f16((64,), -1, 1, 7202)
    inst = capi.INSTANCE_AUTO if auto else _stem(capi.OP_CONV2D_FWD_F16)
    out = _conv(inp, wei, bias, None, S, D, P, inst)
    _f16_close(out, lit.conv2d_fwd_bias_relu_f16(inp, wei, bias, None, S, D, P))
    assert (out >= 0).all() and (out == 0).any()


def test_stem_instance_refuses_other_layers():
    op = ck.DeviceConv2dFwdF16(_stem(capi.OP_CONV2D_FWD_F16))
    ok = op.MakeArgumentPointer(0, 0, 0, 2, 64, 3, [32, 32], [7, 7], [16, 16], [2, 2], [1, 1], [3, 3], [3, 3], None, None, None)
    assert op.IsSupportedArgument(ok)
    for bad in [
        op.MakeArgumentPointer(0, 0, 0, 2, 64, 4, [32, 32], [7, 7], [16, 16], [2, 2], [1, 1], [3, 3], [3, 3], None, None, None),
        op.MakeArgumentPointer(0, 0, 0, 2, 32, 3, [32, 32], [7, 7], [16, 16], [2, 2], [1, 1], [3, 3], [3, 3], None, None, None),
        op.MakeArgumentPointer(0, 0, 0, 2, 64, 3, [32, 32], [7, 7], [32, 32], [1, 1], [1, 1], [3, 3], [3, 3], None, None, None),
        op.MakeArgumentPointer(0, 0, 0, 2, 64, 3, [32, 32], [5, 5], [16, 16], [2, 2], [1, 1], [2, 2], [2, 2], None, None, None),
    ]:
        assert not op.IsSupportedArgument(bad)
