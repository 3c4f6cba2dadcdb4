"""ctypes binding of libck_oracle.so (oracle/ck_oracle.cpp). Test infrastructure."""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libck_oracle.so")

EPI_PASSTHROUGH = 0
EPI_REQUANT_CK = 1   # example-14 functor, literal (no rounding, truncating cast)
EPI_REQUANT_RND = 2  # clamp(rint(sR * relu(clamp(rint(sG * acc)))))

_lib = None


def build(force=False):
    """Compile the oracle with the host compiler (seconds)."""
    src = os.path.join(_HERE, "ck_oracle.cpp")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libck_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.cko_half_to_float.restype = C.c_float
        _lib.cko_half_to_float.argtypes = [C.c_uint16]
        _lib.cko_float_to_half.restype = C.c_uint16
        _lib.cko_float_to_half.argtypes = [C.c_float]
        _lib.cko_epilogue_i8.restype = C.c_int8
        _lib.cko_epilogue_i8.argtypes = [C.c_int32, C.c_int, C.c_float, C.c_float]
        _lib.cko_mul2_clamp.restype = C.c_int8
        _lib.cko_mul2_clamp.argtypes = [C.c_int32, C.c_float, C.c_int]
        _lib.cko_fast_gelu.restype = C.c_float
        _lib.cko_fast_gelu.argtypes = [C.c_float]
        _lib.cko_conv_out_len.restype = C.c_int
        _lib.cko_magic_division_divide.restype = C.c_uint32
        _lib.cko_magic_division_divide.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32]
        _lib.cko_check_err_f16.restype = C.c_int64
        _lib.cko_check_err_i8.restype = C.c_int64
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _i64(*xs):
    return [C.c_int64(int(x)) for x in xs]


def hardware_threads():
    return int(lib().cko_hardware_threads())


def _estrides(a):
    return [s // a.itemsize for s in a.strides]


def gemm_i8(a_mk, b_kn, epi=EPI_PASSTHROUGH, scale_gemm=1.0, scale_relu=1.0, acc_float=None, nthreads=0):
    """a_mk: int8 [M,K] view, b_kn: int8 [K,N] view (any strides). Returns int8 [M,N] row-major."""
    assert a_mk.dtype == np.int8 and b_kn.dtype == np.int8
    M, K = a_mk.shape
    K2, N = b_kn.shape
    assert K == K2
    if acc_float is None:
        acc_float = epi != EPI_PASSTHROUGH
    c = np.empty((M, N), np.int8)
    sa, sb = _estrides(a_mk), _estrides(b_kn)
    lib().cko_gemm_i8(_p(a_mk), _p(b_kn), _p(c), M, N, K, *_i64(sa[0], sa[1], sb[0], sb[1], N, 1),
                      int(bool(acc_float)), int(epi), C.c_float(scale_gemm), C.c_float(scale_relu),
                      int(nthreads))
    return c


def gemm_i8_acc(a_mk, b_kn, nthreads=0):
    M, K = a_mk.shape
    _, N = b_kn.shape
    acc = np.empty((M, N), np.int32)
    sa, sb = _estrides(a_mk), _estrides(b_kn)
    lib().cko_gemm_i8_acc(_p(a_mk), _p(b_kn), _p(acc), M, N, K, *_i64(sa[0], sa[1], sb[0], sb[1]),
                          int(nthreads))
    return acc


def gemm_f16(a_mk, b_kn, nthreads=0):
    assert a_mk.dtype == np.float16 and b_kn.dtype == np.float16
    M, K = a_mk.shape
    _, N = b_kn.shape
    c = np.empty((M, N), np.float16)
    sa, sb = _estrides(a_mk), _estrides(b_kn)
    lib().cko_gemm_f16(_p(a_mk), _p(b_kn), _p(c), M, N, K, *_i64(sa[0], sa[1], sb[0], sb[1], N, 1),
                       int(nthreads))
    return c


def float_to_bf16(x):
    """float32 array -> uint16 array of bfloat16 bit patterns (the reference's round-to-nearest-even)."""
    lib().cko_float_to_bf16.restype = C.c_uint16
    lib().cko_float_to_bf16.argtypes = [C.c_float]
    flat = np.asarray(x, np.float32).ravel()
    return np.array([lib().cko_float_to_bf16(float(v)) for v in flat], np.uint16).reshape(np.shape(x))


def gemm_bf16(a_mk, b_kn, nthreads=0):
    """a, b: uint16 arrays of bfloat16 bit patterns; returns uint16 [M,N]."""
    M, K = a_mk.shape
    _, N = b_kn.shape
    c = np.empty((M, N), np.uint16)
    lib().cko_gemm_bf16(_p(a_mk), _p(b_kn), _p(c), M, N, K, *_i64(*_estrides(a_mk)), *_i64(*_estrides(b_kn)),
                        *_i64(N, 1), int(nthreads))
    return c


def batched_gemm_f16(a_gmk, b_gkn, nthreads=0):
    G, M, K = a_gmk.shape
    _, _, N = b_gkn.shape
    c = np.empty((G, M, N), np.float16)
    sa, sb = _estrides(a_gmk), _estrides(b_gkn)
    lib().cko_batched_gemm_f16(_p(a_gmk), _p(b_gkn), _p(c), G, M, N, K, *_i64(*sa, *sb, M * N, N, 1),
                               int(nthreads))
    return c


def batched_gemm_gemm_f16(a_gmk, b0_gkn, b1_gno, nthreads=0):
    G, M, K = a_gmk.shape
    _, _, N = b0_gkn.shape
    _, _, O = b1_gno.shape
    c = np.empty((G, M, O), np.float16)
    sa, sb0, sb1 = _estrides(a_gmk), _estrides(b0_gkn), _estrides(b1_gno)
    lib().cko_batched_gemm_gemm_f16(_p(a_gmk), _p(b0_gkn), _p(b1_gno), _p(c), G, M, N, K, O,
                                    *_i64(*sa, *sb0, *sb1, M * O, O, 1), int(nthreads))
    return c


def batched_gemm_softmax_gemm_f16(a_gmk, b0_gkn, b1_gno, scale=1.0, mask_upper=False, nthreads=0):
    """C[g] = half(half(softmax_n(mask(scale * A[g] B0[g]))) B1[g]); mask_upper: scores with n > m are masked."""
    G, M, K = a_gmk.shape
    _, _, N = b0_gkn.shape
    _, _, O = b1_gno.shape
    c = np.empty((G, M, O), np.float16)
    sa, sb0, sb1 = _estrides(a_gmk), _estrides(b0_gkn), _estrides(b1_gno)
    lib().cko_batched_gemm_softmax_gemm_f16(_p(a_gmk), _p(b0_gkn), _p(b1_gno), _p(c), G, M, N, K, O,
                                            *_i64(*sa, *sb0, *sb1, M * O, O, 1), C.c_float(scale),
                                            int(bool(mask_upper)), int(nthreads))
    return c


def conv_out_len(in_len, filt, stride, dil, pl, pr):
    return int(lib().cko_conv_out_len(in_len, filt, stride, dil, pl, pr))


def conv2d_fwd(inp_nhwc, wei_kyxc, strides=(1, 1), dilations=(1, 1), pads=(0, 0), right_pads=None,
               epi=EPI_PASSTHROUGH, scale_gemm=1.0, scale_relu=1.0, nthreads=0):
    """NHWC input, KYXC weights -> NHWK output; dtype float32 / float16 / int8."""
    inp = np.ascontiguousarray(inp_nhwc)
    wei = np.ascontiguousarray(wei_kyxc)
    N, Hi, Wi, Cc = inp.shape
    K, Y, X, C2 = wei.shape
    assert Cc == C2
    if right_pads is None:
        right_pads = pads
    Ho = conv_out_len(Hi, Y, strides[0], dilations[0], pads[0], right_pads[0])
    Wo = conv_out_len(Wi, X, strides[1], dilations[1], pads[1], right_pads[1])
    out = np.empty((N, Ho, Wo, K), inp.dtype)
    args = [_p(inp), _p(wei), _p(out), N, K, Cc, Hi, Wi, Y, X, Ho, Wo, strides[0], strides[1],
            dilations[0], dilations[1], pads[0], pads[1]]
    if inp.dtype == np.float32:
        lib().cko_conv2d_fwd_f32(*args, int(nthreads))
    elif inp.dtype == np.float16:
        lib().cko_conv2d_fwd_f16(*args, int(nthreads))
    elif inp.dtype == np.int8:
        lib().cko_conv2d_fwd_i8(*args, int(epi), C.c_float(scale_gemm), C.c_float(scale_relu),
                                int(nthreads))
    else:
        raise TypeError(inp.dtype)
    return out


def convnd_fwd(inp, wei, strides, dilations, pads, right_pads=None, epi=EPI_PASSTHROUGH, scale_gemm=1.0,
               scale_relu=1.0, nthreads=0):
    """Forward convolution with 1, 2 or 3 spatial dimensions: N(D)(H)WC input, K(Z)(Y)XC weights ->
    N(D)(H)WK output; dtype float32 / float16 / int8. Missing leading dimensions have extent 1."""
    inp = np.ascontiguousarray(inp)
    wei = np.ascontiguousarray(wei)
    nd = inp.ndim - 2
    assert nd in (1, 2, 3) and wei.ndim == inp.ndim and len(strides) == len(dilations) == len(pads) == nd
    if right_pads is None:
        right_pads = pads
    lead = 3 - nd
    in_len = [1] * lead + list(inp.shape[1:-1])
    filt = [1] * lead + list(wei.shape[1:-1])
    st = [1] * lead + list(strides)
    dl = [1] * lead + list(dilations)
    pl = [0] * lead + list(pads)
    pr = [0] * lead + list(right_pads)
    out_len = [conv_out_len(in_len[i], filt[i], st[i], dl[i], pl[i], pr[i]) for i in range(3)]
    N, Cc, K = inp.shape[0], inp.shape[-1], wei.shape[0]
    assert wei.shape[-1] == Cc
    out = np.empty((N, *out_len[lead:], K), inp.dtype)
    arr = lambda v: (C.c_int * 3)(*[int(x) for x in v])
    args = [_p(inp), _p(wei), _p(out), N, K, Cc, arr(in_len), arr(filt), arr(out_len), arr(st), arr(dl), arr(pl)]
    if inp.dtype == np.float32:
        lib().cko_conv3d_fwd_f32(*args, int(nthreads))
    elif inp.dtype == np.float16:
        lib().cko_conv3d_fwd_f16(*args, int(nthreads))
    elif inp.dtype == np.int8:
        lib().cko_conv3d_fwd_i8(*args, int(epi), C.c_float(scale_gemm), C.c_float(scale_relu), int(nthreads))
    else:
        raise TypeError(inp.dtype)
    return out


def conv2d_fwd_bias_relu_f16(inp_nhwc, wei_kyxc, bias_k, resi_nhwk=None, strides=(1, 1), dilations=(1, 1),
                             pads=(0, 0), right_pads=None, nthreads=0):
    """conv + bias + ReLU (+ residual), fp16 tensors, fp32 through the functor, one rounding."""
    inp = np.ascontiguousarray(inp_nhwc, np.float16)
    wei = np.ascontiguousarray(wei_kyxc, np.float16)
    bias = np.ascontiguousarray(bias_k, np.float16)
    N, Hi, Wi, Cc = inp.shape
    K, Y, X, _ = wei.shape
    if right_pads is None:
        right_pads = pads
    Ho = conv_out_len(Hi, Y, strides[0], dilations[0], pads[0], right_pads[0])
    Wo = conv_out_len(Wi, X, strides[1], dilations[1], pads[1], right_pads[1])
    out = np.empty((N, Ho, Wo, K), np.float16)
    resi = None if resi_nhwk is None else np.ascontiguousarray(resi_nhwk, np.float16)
    assert resi is None or resi.shape == out.shape
    lib().cko_conv2d_fwd_bias_relu_f16(_p(inp), _p(wei), _p(bias), _p(resi) if resi is not None else None,
                                       _p(out), N, K, Cc, Hi, Wi, Y, X, Ho, Wo, strides[0], strides[1],
                                       dilations[0], dilations[1], pads[0], pads[1], int(nthreads))
    return out


def gemm_f16_add_relu(a_mk, b_kn, d_mn, nthreads=0):
    """E = relu(half(half(A*B) + D)) as example 03 verifies it; d_mn may be a broadcast view."""
    M, K = a_mk.shape
    _, N = b_kn.shape
    d = np.broadcast_to(d_mn, (M, N))
    e = np.empty((M, N), np.float16)
    lib().cko_gemm_f16_add_relu(_p(a_mk), _p(b_kn), _p(d), _p(e), M, N, K, *_i64(*_estrides(a_mk)),
                                *_i64(*_estrides(b_kn)), *_i64(*_estrides(d)), *_i64(N, 1), int(nthreads))
    return e


def gemm_f16_bilinear(a_mk, b_kn, d_mn, alpha, beta, nthreads=0):
    """E = half(alpha * (A*B) + beta * D) as example 02 verifies it: one rounding, of the fp32 result."""
    M, K = a_mk.shape
    _, N = b_kn.shape
    d = np.broadcast_to(d_mn, (M, N))
    e = np.empty((M, N), np.float16)
    lib().cko_gemm_f16_bilinear(_p(a_mk), _p(b_kn), _p(d), _p(e), M, N, K, *_i64(*_estrides(a_mk)),
                                *_i64(*_estrides(b_kn)), *_i64(*_estrides(d)), *_i64(N, 1), C.c_float(alpha),
                                C.c_float(beta), int(nthreads))
    return e


def fast_gelu(x):
    """element_wise::FastGelu on one float, as written in the reference."""
    return float(lib().cko_fast_gelu(float(x)))


def gemm_f16_add_add_fastgelu(a_mk, b_kn, d0_mn, d1_mn, nthreads=0):
    """E = half(fast_gelu(A*B + D0 + D1)) as example 04 verifies it; D0 / D1 may be broadcast views."""
    M, K = a_mk.shape
    _, N = b_kn.shape
    d0 = np.broadcast_to(d0_mn, (M, N))
    d1 = np.broadcast_to(d1_mn, (M, N))
    e = np.empty((M, N), np.float16)
    lib().cko_gemm_f16_add_add_fastgelu(_p(a_mk), _p(b_kn), _p(d0), _p(d1), _p(e), M, N, K, *_i64(*_estrides(a_mk)),
                                        *_i64(*_estrides(b_kn)), *_i64(*_estrides(d0)), *_i64(*_estrides(d1)),
                                        *_i64(N, 1), int(nthreads))
    return e


def epilogue_i8(acc, epi, scale_gemm, scale_relu):
    return int(lib().cko_epilogue_i8(int(acc), int(epi), C.c_float(scale_gemm), C.c_float(scale_relu)))


def mul2_clamp(acc, requant_scale, relu):
    """Activation_Mul2_Clamp<PassThrough / Relu> on one accumulator (upstream functor, literal restatement)."""
    return int(lib().cko_mul2_clamp(int(acc), C.c_float(requant_scale), int(bool(relu))))


def gemm_i8_mul2_clamp(a_mk, b_kn, scales_n, relu, nthreads=0):
    """int8 GEMM with int32 accumulation and one requant scale per output column, element by element."""
    acc = gemm_i8_acc(a_mk, b_kn, nthreads)
    out = np.empty(acc.shape, np.int8)
    for m in range(acc.shape[0]):
        for n in range(acc.shape[1]):
            out[m, n] = mul2_clamp(acc[m, n], scales_n[n], relu)
    return out


def magic_params(d):
    m, s = C.c_uint32(), C.c_uint32()
    lib().cko_magic_division_params(C.c_uint32(d), C.byref(m), C.byref(s))
    return m.value, s.value


def magic_divide(n, mult, shift):
    return int(lib().cko_magic_division_divide(n, mult, shift))


def check_err_f16(out, ref, rtol=1e-3, atol=1e-3):
    """Returns (n_bad, max_err) under the reference comparator |o-r| <= atol + rtol*|r|."""
    out = np.ascontiguousarray(out, np.float16)
    ref = np.ascontiguousarray(ref, np.float16)
    assert out.shape == ref.shape
    me = C.c_double()
    bad = lib().cko_check_err_f16(_p(out), _p(ref), C.c_int64(out.size), C.c_double(rtol),
                                  C.c_double(atol), C.byref(me))
    return int(bad), float(me.value)
