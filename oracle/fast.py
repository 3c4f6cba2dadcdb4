"""numpy forms of the oracle for full-size checks. Test infrastructure.

int8 products summed in fp32 stay exact while sum(|a*b|) < 2**24, so an fp32
BLAS GEMM on int8-valued floats returns the exact integer accumulators in any
summation order (asserted below). The epilogue is the reference functor written
with numpy float32 ufuncs: each ufunc rounds once, nothing is fused.
Equality of these forms with the literal restatement (oracle.lit) on small
shapes is asserted in tests/test_oracle.py.
"""
import numpy as np

from .lit import EPI_PASSTHROUGH, EPI_REQUANT_CK, EPI_REQUANT_RND


def epilogue_i8(acc_i32, epi, scale_gemm=1.0, scale_relu=1.0):
    acc_i32 = np.asarray(acc_i32)
    if epi == EPI_PASSTHROUGH:
        return (acc_i32.astype(np.int64) & 0xFF).astype(np.uint8).view(np.int8)
    x = acc_i32.astype(np.float32)
    sg, sr = np.float32(scale_gemm), np.float32(scale_relu)
    lo, hi = np.float32(-128), np.float32(127)
    if epi == EPI_REQUANT_CK:
        g = sg * x
        r = np.where(g > 0, g, np.float32(0))
        q = sr * r
        y = np.where(q > hi, hi, np.where(q < lo, lo, q))
    elif epi == EPI_REQUANT_RND:
        t = np.rint(sg * x)
        t = np.where(t > hi, hi, np.where(t < lo, lo, t))
        r = np.where(t > 0, t, np.float32(0))
        u = np.rint(sr * r)
        y = np.where(u > hi, hi, np.where(u < lo, lo, u))
    else:
        raise ValueError(epi)
    assert y.dtype == np.float32
    return y.astype(np.int32).astype(np.int8)  # truncation toward zero; in range after the clamp


def epilogue_i8_mul2_clamp(acc_i32, scales, relu):
    """Activation_Mul2_Clamp over a [.., N] accumulator array with N scales (numpy float32 ufuncs, one rounding each)."""
    x = np.asarray(acc_i32).astype(np.float32)
    if relu:
        x = np.where(x > 0, x, np.float32(0))
    y = np.asarray(scales, np.float32) * x
    lo, hi = np.float32(-128), np.float32(127)
    y = np.minimum(np.maximum(y, lo), hi)
    assert y.dtype == np.float32
    return y.astype(np.int32).astype(np.int8)


def gemm_i8_acc(a_mk, b_kn):
    a = np.asarray(a_mk)
    b = np.asarray(b_kn)
    bound = int(np.abs(a).max(initial=0)) * int(np.abs(b).max(initial=0)) * a.shape[1]
    assert bound < 2 ** 24, "fp32 BLAS would not be exact for these magnitudes"
    acc = a.astype(np.float32) @ b.astype(np.float32)
    return acc.astype(np.int32)


def gemm_i8(a_mk, b_kn, epi=EPI_PASSTHROUGH, scale_gemm=1.0, scale_relu=1.0):
    return epilogue_i8(gemm_i8_acc(a_mk, b_kn), epi, scale_gemm, scale_relu)


def gemm_f16(a_mk, b_kn):
    """fp32-accumulated product rounded once to fp16 (BLAS summation order)."""
    return (np.asarray(a_mk, np.float32) @ np.asarray(b_kn, np.float32)).astype(np.float16)


def bf16_to_f32(u16):
    """uint16 bfloat16 bit patterns -> float32."""
    return (np.asarray(u16, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(x):
    """float32 -> uint16 bfloat16 bit patterns, round to nearest even (finite inputs)."""
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


def gemm_bf16(a_mk, b_kn):
    """fp32-accumulated product of bf16 operands rounded once to bf16 (BLAS summation order)."""
    return f32_to_bf16(bf16_to_f32(a_mk) @ bf16_to_f32(b_kn))


def im2col(inp_nhwc, Y, X, strides, dilations, pads, right_pads=None):
    """[N,Hi,Wi,C] -> [N*Ho*Wo, Y*X*C] with (y,x,c) ordering, c fastest; zero padding."""
    if right_pads is None:
        right_pads = pads
    N, Hi, Wi, C = inp_nhwc.shape
    sH, sW = strides
    dH, dW = dilations
    Ho = (Hi + pads[0] + right_pads[0] - ((Y - 1) * dH + 1)) // sH + 1
    Wo = (Wi + pads[1] + right_pads[1] - ((X - 1) * dW + 1)) // sW + 1
    p = np.zeros((N, Hi + pads[0] + right_pads[0], Wi + pads[1] + right_pads[1], C), inp_nhwc.dtype)
    p[:, pads[0]:pads[0] + Hi, pads[1]:pads[1] + Wi, :] = inp_nhwc
    cols = np.empty((N, Ho, Wo, Y, X, C), inp_nhwc.dtype)
    for y in range(Y):
        for x in range(X):
            cols[:, :, :, y, x, :] = p[:, y * dH:y * dH + (Ho - 1) * sH + 1:sH,
                                       x * dW:x * dW + (Wo - 1) * sW + 1:sW, :]
    return cols.reshape(N * Ho * Wo, Y * X * C), Ho, Wo


def im2col_nd(inp, filt, strides, dilations, pads, right_pads=None):
    """[N, (D,) (H,) W, C] -> [N * prod(out), prod(filt) * C], taps slowest-dimension first, c fastest."""
    nd = inp.ndim - 2
    if right_pads is None:
        right_pads = pads
    lead = 3 - nd
    x = inp.reshape(inp.shape[0], *([1] * lead), *inp.shape[1:])
    f = [1] * lead + list(filt)
    s = [1] * lead + list(strides)
    d = [1] * lead + list(dilations)
    pl = [0] * lead + list(pads)
    pr = [0] * lead + list(right_pads)
    N, Cc = x.shape[0], x.shape[-1]
    o = [(x.shape[1 + i] + pl[i] + pr[i] - ((f[i] - 1) * d[i] + 1)) // s[i] + 1 for i in range(3)]
    p = np.zeros((N, *[x.shape[1 + i] + pl[i] + pr[i] for i in range(3)], Cc), inp.dtype)
    p[:, pl[0]:pl[0] + x.shape[1], pl[1]:pl[1] + x.shape[2], pl[2]:pl[2] + x.shape[3], :] = x
    cols = np.empty((N, *o, *f, Cc), inp.dtype)
    for z in range(f[0]):
        for y in range(f[1]):
            for xx in range(f[2]):
                cols[:, :, :, :, z, y, xx, :] = p[:, z * d[0]:z * d[0] + (o[0] - 1) * s[0] + 1:s[0],
                                                  y * d[1]:y * d[1] + (o[1] - 1) * s[1] + 1:s[1],
                                                  xx * d[2]:xx * d[2] + (o[2] - 1) * s[2] + 1:s[2], :]
    return cols.reshape(N * o[0] * o[1] * o[2], f[0] * f[1] * f[2] * Cc), o[lead:]


def convnd_fwd(inp, wei, strides, dilations, pads, right_pads=None, epi=EPI_PASSTHROUGH, scale_gemm=1.0,
               scale_relu=1.0):
    """N-d forward conv through im2col + BLAS: int8 exact (with the requant epilogues), fp16 in BLAS order."""
    K = wei.shape[0]
    cols, o = im2col_nd(inp, wei.shape[1:-1], strides, dilations, pads, right_pads)
    w = wei.reshape(K, -1).T
    if inp.dtype == np.int8:
        return epilogue_i8(gemm_i8_acc(cols, w), epi, scale_gemm, scale_relu).reshape(inp.shape[0], *o, K)
    return (cols.astype(np.float32) @ w.astype(np.float32)).astype(np.float16).reshape(inp.shape[0], *o, K)


def conv2d_fwd_i8(inp_nhwc, wei_kyxc, strides=(1, 1), dilations=(1, 1), pads=(0, 0), right_pads=None,
                  epi=EPI_PASSTHROUGH, scale_gemm=1.0, scale_relu=1.0):
    N = inp_nhwc.shape[0]
    K, Y, X, C = wei_kyxc.shape
    cols, Ho, Wo = im2col(inp_nhwc, Y, X, strides, dilations, pads, right_pads)
    acc = gemm_i8_acc(cols, wei_kyxc.reshape(K, Y * X * C).T)
    return epilogue_i8(acc, epi, scale_gemm, scale_relu).reshape(N, Ho, Wo, K)


def gemm_i8_mul2_clamp(a_mk, b_kn, scales, relu):
    return epilogue_i8_mul2_clamp(gemm_i8_acc(a_mk, b_kn), scales, relu)


def conv2d_fwd_i8_mul2_clamp(inp_nhwc, wei_kyxc, scales_k, relu, strides=(1, 1), dilations=(1, 1), pads=(0, 0),
                             right_pads=None):
    N = inp_nhwc.shape[0]
    K, Y, X, C = wei_kyxc.shape
    cols, Ho, Wo = im2col(inp_nhwc, Y, X, strides, dilations, pads, right_pads)
    acc = gemm_i8_acc(cols, wei_kyxc.reshape(K, Y * X * C).T)
    return epilogue_i8_mul2_clamp(acc, scales_k, relu).reshape(N, Ho, Wo, K)


def conv2d_fwd_f16(inp_nhwc, wei_kyxc, strides=(1, 1), dilations=(1, 1), pads=(0, 0), right_pads=None):
    N = inp_nhwc.shape[0]
    K, Y, X, C = wei_kyxc.shape
    cols, Ho, Wo = im2col(inp_nhwc, Y, X, strides, dilations, pads, right_pads)
    out = cols.astype(np.float32) @ wei_kyxc.reshape(K, Y * X * C).T.astype(np.float32)
    return out.astype(np.float16).reshape(N, Ho, Wo, K)


def conv2d_fwd_bias_relu_f16(inp_nhwc, wei_kyxc, bias_k, resi_nhwk=None, strides=(1, 1), dilations=(1, 1),
                             pads=(0, 0), right_pads=None):
    """conv + bias + ReLU (+ residual) in fp32, rounded once to fp16 (BLAS summation order)."""
    N = inp_nhwc.shape[0]
    K, Y, X, C = wei_kyxc.shape
    cols, Ho, Wo = im2col(inp_nhwc, Y, X, strides, dilations, pads, right_pads)
    acc = cols.astype(np.float32) @ wei_kyxc.reshape(K, Y * X * C).T.astype(np.float32)
    y = np.maximum(acc + np.asarray(bias_k, np.float32)[None, :], np.float32(0))
    if resi_nhwk is not None:
        y = y + np.asarray(resi_nhwk, np.float32).reshape(-1, K)
    return y.astype(np.float16).reshape(N, Ho, Wo, K)


def gemm_f16_add_relu(a_mk, b_kn, d_mn):
    """relu(half(half(A*B) + D)): the GEMM result is rounded to fp16 before the functor."""
    c = (np.asarray(a_mk, np.float32) @ np.asarray(b_kn, np.float32)).astype(np.float16)
    x = (c.astype(np.float32) + np.asarray(d_mn, np.float32)).astype(np.float16)
    return np.maximum(x, np.float16(0))


def gemm_f16_bilinear(a_mk, b_kn, d_mn, alpha, beta):
    """half(alpha * (A*B) + beta * D) on the fp32 product (fp32 BLAS sums: within tolerance of the literal form)."""
    acc = np.asarray(a_mk, np.float32) @ np.asarray(b_kn, np.float32)
    return (np.float32(alpha) * acc + np.float32(beta) * np.asarray(d_mn, np.float32)).astype(np.float16)


def fast_gelu(x):
    """element_wise::FastGelu in fp32 on an array, written as the reference writes it."""
    x = np.asarray(x, np.float32)
    with np.errstate(over="ignore"):
        u = np.float32(2) * x * (np.float32(0.035677) * x * x + np.float32(0.797885))
        emu = np.exp(-u)
        cdf = np.float32(0.5) + np.float32(0.5) * (np.float32(2) / (np.float32(1) + emu) - np.float32(1))
    return x * cdf


def gemm_f16_add_add_fastgelu(a_mk, b_kn, d0_mn, d1_mn):
    acc = np.asarray(a_mk, np.float32) @ np.asarray(b_kn, np.float32)
    return fast_gelu(acc + np.asarray(d0_mn, np.float32) + np.asarray(d1_mn, np.float32)).astype(np.float16)


def batched_gemm_gemm_f16(a_gmk, b0_gkn, b1_gno):
    s = np.matmul(np.asarray(a_gmk, np.float32), np.asarray(b0_gkn, np.float32)).astype(np.float16)
    return np.matmul(s.astype(np.float32), np.asarray(b1_gno, np.float32)).astype(np.float16)


def batched_gemm_softmax_gemm_f16(a_gmk, b0_gkn, b1_gno, scale=1.0, mask_upper=False):
    """numpy form of lit.batched_gemm_softmax_gemm_f16 (fp32 BLAS sums: within tolerance, not bit-equal)."""
    x = np.float32(scale) * np.matmul(np.asarray(a_gmk, np.float32), np.asarray(b0_gkn, np.float32))
    if mask_upper:
        M, N = x.shape[1:]
        x = np.where(np.arange(N)[None, None, :] > np.arange(M)[None, :, None], -np.inf, x).astype(np.float32)
    e = np.exp(x - x.max(axis=2, keepdims=True))
    p = (e / e.sum(axis=2, keepdims=True, dtype=np.float32)).astype(np.float16)
    return np.matmul(p.astype(np.float32), np.asarray(b1_gno, np.float32)).astype(np.float16)
