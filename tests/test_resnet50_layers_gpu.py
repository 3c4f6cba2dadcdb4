"""Every layer of the reference's whole-network script (script/profile_resnet50.sh:24-46, run there as ckProfiler
conv_fwd / conv_fwd_bias_relu / conv_fwd_bias_relu_add at N = 256) at a small batch through the automatic instance
choice against the CPU oracle: int8 + rounded requant bit-exact, fp16 within rtol = atol = 1e-2, the fused forms of
the script's second half against ReferenceConvFwd_Bias_Activation[_Add] restated."""
import numpy as np
import pytest

import bench
import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8
from oracle import fast, lit

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2
N = 2


def _geom(layer):
    K, C, f, HW, st, pd = layer
    return K, C, f, HW, (st, st), (1, 1), (pd, pd)


@pytest.mark.parametrize("layer", bench.RESNET50_LAYERS)
def test_resnet50_layer_int8_bit_exact(layer):
    import gpu_util
    K, C, f, HW, s, d, p = _geom(layer)
    inp = uniform_int8((N, HW, HW, C), -5, 5, 8000 + C)
    wei = uniform_int8((K, f, f, C), -5, 5, 8001 + K)
    rq = ck.RequantReluRequant(0.01, 0.5, rounded=True)
    out = gpu_util.conv2d_fwd(inp, wei, s, d, p, out_op=rq)
    np.testing.assert_array_equal(out, fast.conv2d_fwd_i8(inp, wei, s, d, p, epi=lit.EPI_REQUANT_RND, scale_gemm=0.01, scale_relu=0.5))


@pytest.mark.parametrize("layer", bench.RESNET50_LAYERS)
def test_resnet50_layer_fp16_plain_and_fused(layer):
    import gpu_util
    from test_fused_epilogue_gpu import _conv
    K, C, f, HW, s, d, p = _geom(layer)
    inp = uniform_f16((N, HW, HW, C), -1, 1, 8100 + C)
    wei = uniform_f16((K, f, f, C), -1, 1, 8101 + K)
    bias = uniform_f16((K,), -1, 1, 8102)

    def close(out, ref):
        bad, max_err = lit.check_err_f16(out, ref, RTOL, ATOL)
        assert bad == 0, f"{bad} outside tolerance, max err {max_err}"
    close(gpu_util.conv2d_fwd(inp, wei, s, d, p), fast.conv2d_fwd_f16(inp, wei, s, d, p))
    close(_conv(inp, wei, bias, None, s, d, p), fast.conv2d_fwd_bias_relu_f16(inp, wei, bias, None, s, d, p))
    if layer in bench.RESNET50_BIAS_RELU_ADD:
        Ho = (HW + 2 * p[0] - f) // s[0] + 1
        resi = uniform_f16((N, Ho, Ho, K), -1, 1, 8103)
        close(_conv(inp, wei, bias, resi, s, d, p), fast.conv2d_fwd_bias_relu_f16(inp, wei, bias, resi, s, d, p))
