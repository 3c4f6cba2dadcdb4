"""GPU parity: conv forward with one and three spatial dimensions (NWC / NDHWC) through the C ABI against the
CPU oracle.

Parameter sets follow the reference's test/convnd_fwd/conv1d_fwd.cpp:73-78,94 and conv3d_fwd.cpp:76-81,97
(default 3-tap stride 2 dilation 2 pad 2; 1-tap stride 1 pad 0; 1-tap stride 2 pad 0; the 18^3 / 36 cases of the
IntegerValues tests), its golden vectors (test/reference_conv_fwd/reference_conv_fwd.cpp:156-392) and its
refusals of tensors above 2 GB (conv3d_fwd.cpp:160-277). int8 is bit-exact; fp16 within rtol = atol = 1e-2.
"""
import ctypes as C
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

# (input shape N (D) (H) W C, weight shape K (Z) (Y) X C, strides, dilations, pads)
SMALL = [
    ((2, 9, 16), (32, 3, 16), (2,), (2,), (2,)),                                  # 1-D "default" family
    ((3, 28, 32), (48, 1, 32), (1,), (1,), (0,)),                                 # 1-D filter 1, stride 1, pad 0
    ((2, 28, 32), (16, 1, 32), (2,), (1,), (0,)),                                 # 1-D filter 1, pad 0
    ((2, 6, 7, 5, 16), (32, 3, 3, 3, 16), (2, 2, 2), (2, 2, 2), (2, 2, 2)),       # 3-D "default" family
    ((2, 5, 6, 7, 32), (48, 1, 1, 1, 32), (1, 1, 1), (1, 1, 1), (0, 0, 0)),       # 3-D 1x1x1, stride 1 (runs as 2-D)
    ((2, 5, 6, 7, 32), (16, 1, 1, 1, 32), (2, 2, 2), (1, 1, 1), (0, 0, 0)),       # 3-D 1x1x1, stride 2
    ((1, 4, 9, 5, 16), (80, 2, 3, 2, 16), (1, 2, 1), (2, 1, 1), (1, 0, 1)),       # asymmetric everything
    ((3, 3, 4, 4, 48), (24, 3, 1, 3, 48), (1, 1, 1), (1, 1, 1), (1, 0, 1)),       # depth taps, C not a multiple of the K tile
    ((2, 4, 6, 6, 16), (32, 1, 3, 3, 16), (1, 1, 1), (1, 1, 1), (0, 1, 1)),       # unconvolved depth: N * D images of a 2-D conv
]


def _f16_close(out, ref):
    bad, max_err = lit.check_err_f16(out, ref, RTOL, ATOL)
    assert bad == 0, f"{bad} outside tolerance, max err {max_err}"


@pytest.mark.parametrize("case", SMALL)
@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 0, 2, 4, 6, 8])
def test_convnd_int8_small_cases_bit_exact(case, instance):
    import gpu_util
    si, sw, s, d, p = case
    inp = uniform_int8(si, -5, 5, 1100 + si[-1])
    wei = uniform_int8(sw, -5, 5, 1200 + sw[0])
    out = gpu_util.convnd_fwd(inp, wei, s, d, p, instance=instance)
    np.testing.assert_array_equal(out, lit.convnd_fwd(inp, wei, s, d, p))
    rq = ck.RequantReluRequant(0.05, 0.7, rounded=True)
    out = gpu_util.convnd_fwd(inp, wei, s, d, p, out_op=rq, instance=instance)
    np.testing.assert_array_equal(
        out, lit.convnd_fwd(inp, wei, s, d, p, epi=lit.EPI_REQUANT_RND, scale_gemm=0.05, scale_relu=0.7))
    assert out.max() > 0


@pytest.mark.parametrize("case", SMALL)
@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 1, 3, 5, 7])
def test_convnd_fp16_small_cases(case, instance):
    import gpu_util
    si, sw, s, d, p = case
    inp = uniform_f16(si, -1, 1, 1300 + si[-1])
    wei = uniform_f16(sw, -1, 1, 1400 + sw[0])
    _f16_close(gpu_util.convnd_fwd(inp, wei, s, d, p, instance=instance), lit.convnd_fwd(inp, wei, s, d, p))


GOLD_ND = json.load(open(os.path.join(HERE, "golden", "reference_convnd_fwd_vectors.json")))


@pytest.mark.parametrize("case", [c for c in GOLD_ND["cases"] if c["fill_start_step"] == [0.0, 1.0]],
                         ids=lambda c: c["name"])
def test_convnd_reference_golden_vectors_fp16(case):
    """The reference's golden cases with integer inputs: exactly representable in fp16. Run with the case's own
    channel count (C = 2: the element-wise instance) and with C padded to a whole 16-byte vector by zero channels,
    which add nothing (the vectorised instances)."""
    import gpu_util
    N, K, Cc = case["N"], case["K"], case["C"]
    sp, filt = case["input"], case["filter"]
    for cpad in (Cc, 8):
        inp = np.zeros((N, *sp, cpad), np.float16)
        inp[..., :Cc] = np.arange(N * int(np.prod(sp)) * Cc, dtype=np.float32).reshape(N, *sp, Cc)
        wei = np.zeros((K, *filt, cpad), np.float16)
        wei[..., :Cc] = 0.5
        out = gpu_util.convnd_fwd(inp, wei, case["strides"], case["dilations"], case["left_pads"],
                                  right_pads=case["right_pads"])
        np.testing.assert_array_equal(out.ravel().astype(np.float32), np.array(case["expected"], np.float32))


@pytest.mark.parametrize("dtype", ["i8", "f16"])
@pytest.mark.parametrize("case", [
    ((4, 71, 64), (256, 3, 64), (2,), (2,), (2,)),                                     # conv1d_fwd.cpp:73-74
    ((4, 36, 64), (256, 3, 64), (1,), (2,), (2,)),                                     # conv1d_fwd.cpp:94
    ((4, 28, 28, 28, 64), (256, 3, 3, 3, 64), (2, 2, 2), (2, 2, 2), (2, 2, 2)),        # conv3d_fwd.cpp:76-77
    ((4, 18, 18, 18, 64), (256, 3, 3, 3, 64), (1, 1, 1), (2, 2, 2), (2, 2, 2)),        # conv3d_fwd.cpp:97-98
    ((4, 28, 28, 28, 64), (256, 1, 1, 1, 64), (2, 2, 2), (1, 1, 1), (0, 0, 0)),        # conv3d_fwd.cpp:80-81
])
def test_convnd_reference_test_shapes(case, dtype):
    """The shapes the reference's device tests run, at full size, against the im2col / BLAS form of the oracle
    (bit-exact for int8; the literal loops confirm one image's worth of the fp16 result)."""
    import gpu_util
    si, sw, s, d, p = case
    if dtype == "i8":
        inp, wei = uniform_int8(si, -5, 5, 1500), uniform_int8(sw, -5, 5, 1501)
        out = gpu_util.convnd_fwd(inp, wei, s, d, p, workspace=True)
        np.testing.assert_array_equal(out, fast.convnd_fwd(inp, wei, s, d, p))
    else:
        inp, wei = uniform_f16(si, -1, 1, 1502), uniform_f16(sw, -0.5, 0.5, 1503)
        out = gpu_util.convnd_fwd(inp, wei, s, d, p, workspace=True)
        _f16_close(out, fast.convnd_fwd(inp, wei, s, d, p))
        _f16_close(out[:1, ..., :16], lit.convnd_fwd(inp[:1], wei[:16], s, d, p))


def test_convnd_unsupported_arguments_are_refused():
    """Tensors of 2 GB and more (conv3d_fwd.cpp:160-277), inconsistent output extents, the 2-D specialists asked
    for a 3-D problem."""
    L = capi.lib()
    mk = capi.ConvNdDesc.make

    def out_len(i, f, s, d, p):
        return [(i[k] + 2 * p[k] - ((f[k] - 1) * d[k] + 1)) // s[k] + 1 for k in range(len(i))]

    one = [1, 1, 1]
    for (N, K, Cc, i, f, p) in [(2, 16, 32, [32, 1000, 1000], [3, 3, 3], one),      # input over 2 GB
                                (2, 16, 32, [16, 16, 16], [4, 1000, 1000], one),    # filters over 2 GB
                                (2, 16, 2 * 8, [1000, 1000, 30], [1, 1, 1], [2, 2, 2])]:  # output over 2 GB
        d = mk(N, K, Cc, i, f, out_len(i, f, one, one, p), one, one, p, p)
        assert L.ckx_convnd_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(d), 0, -1) != capi.OK
        arg = ck.DeviceConvNdFwdF16(3).MakeArgumentPointer(0, 0, 0, N, K, Cc, i, f, out_len(i, f, one, one, p), one, one, p, p)
        assert not ck.DeviceConvNdFwdF16(3).IsSupportedArgument(arg)
    ok = mk(2, 16, 16, [6, 6, 6], [3, 3, 3], [4, 4, 4], one, one, [0, 0, 0], [0, 0, 0])
    assert L.ckx_convnd_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(ok), 0, -1) == capi.OK
    assert L.ckx_convnd_fwd_workspace_bytes(capi.OP_CONV2D_FWD_F16, C.byref(ok), -1) >= 0
    bad = mk(2, 16, 16, [6, 6, 6], [3, 3, 3], [4, 5, 4], one, one, [0, 0, 0], [0, 0, 0])
    assert L.ckx_convnd_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(bad), 0, -1) == capi.UNSUPPORTED
    n = L.ckx_num_instances(capi.OP_CONV2D_FWD_F16)
    assert L.ckx_convnd_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(ok), 0, n - 1) == capi.OK           # element-wise
    assert L.ckx_convnd_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(ok), 0, n - 2) == capi.UNSUPPORTED  # pointwise
    assert L.ckx_convnd_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(ok), 0, n - 3) == capi.UNSUPPORTED  # input patch
    assert L.ckx_convnd_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(ok), 0, n) == capi.INVALID_VALUE
    four = capi.ConvNdDesc(4, 1, 16, 16)
    assert L.ckx_convnd_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(four), 0, -1) == capi.INVALID_VALUE
    # fp16 has no requant functor; the operator class refuses vectors of another dimensionality
    assert L.ckx_convnd_fwd_is_supported(capi.OP_CONV2D_FWD_F16, C.byref(ok), capi.EPI_REQUANT_RND, -1) != capi.OK
    with pytest.raises(ValueError):
        ck.DeviceConvNdFwdF16(3).MakeArgumentPointer(0, 0, 0, 1, 16, 16, [6, 6], [3, 3], [4, 4], [1, 1], [1, 1], [0, 0], [0, 0])
    assert len(ck.DeviceConvNdFwdF16.GetInstances(3)) == n
