"""ctypes binding of oracle/_ref/libck_ref.so: the reference's own host operators
(ReferenceGemm / ReferenceConvFwd / ReferenceBatchedGemm) compiled in place by
`make -C oracle ref`. Test infrastructure. The file only exists where it was
built (or travelled with the tree); `load_ref()` returns None otherwise.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_ref", "libck_ref.so")
_REF_TREE = "/root/reference"


def build_ref():
    """Compile the reference host operators where the reference tree is mounted."""
    if os.path.isdir(os.path.join(_REF_TREE, "library", "include")):
        subprocess.check_call(["make", "-C", _HERE, "ref"], stdout=subprocess.DEVNULL)
    return _SO if os.path.exists(_SO) else None


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _es(a):
    return [C.c_long(s // a.itemsize) for s in a.strides]


class _Ref:
    def __init__(self, path):
        self.lib = C.CDLL(path)
        self.lib.ckref_conv_out_len.restype = C.c_int
        self.lib.ckref_magic_division_divide.restype = C.c_uint32
        self.lib.ckref_magic_division_divide.argtypes = [C.c_uint32] * 3

    def gemm_i8_requant(self, a_mk, b_kn, epi, scale_gemm, scale_relu):
        M, K = a_mk.shape
        _, N = b_kn.shape
        c = np.zeros((M, N), np.int8)
        self.lib.ckref_gemm_i8_requant(_p(a_mk), _p(b_kn), _p(c), M, N, K, *_es(a_mk), *_es(b_kn),
                                       C.c_long(N), C.c_long(1), int(epi), C.c_float(scale_gemm),
                                       C.c_float(scale_relu))
        return c

    def gemm_i8(self, a_mk, b_kn):
        M, K = a_mk.shape
        _, N = b_kn.shape
        c = np.zeros((M, N), np.int8)
        self.lib.ckref_gemm_i8(_p(a_mk), _p(b_kn), _p(c), M, N, K, *_es(a_mk), *_es(b_kn), C.c_long(N),
                               C.c_long(1))
        return c

    def gemm_f16(self, a_mk, b_kn):
        M, K = a_mk.shape
        _, N = b_kn.shape
        c = np.zeros((M, N), np.float16)
        self.lib.ckref_gemm_f16(_p(a_mk), _p(b_kn), _p(c), M, N, K, *_es(a_mk), *_es(b_kn), C.c_long(N),
                                C.c_long(1))
        return c

    def batched_gemm_f16(self, a_gmk, b_gkn):
        G, M, K = a_gmk.shape
        _, _, N = b_gkn.shape
        c = np.zeros((G, M, N), np.float16)
        self.lib.ckref_batched_gemm_f16(_p(a_gmk), _p(b_gkn), _p(c), G, M, N, K, *_es(a_gmk),
                                        *_es(b_gkn), C.c_long(M * N), C.c_long(N), C.c_long(1))
        return c

    def batched_gemm_softmax_gemm_f16(self, a_gmk, b0_gkn, b1_gno, scale=1.0, mask_upper=False):
        G, M, K = a_gmk.shape
        _, _, N = b0_gkn.shape
        _, _, O = b1_gno.shape
        c = np.zeros((G, M, O), np.float16)
        self.lib.ckref_batched_gemm_softmax_gemm_f16(_p(a_gmk), _p(b0_gkn), _p(b1_gno), _p(c), G, M, N, K, O,
                                                     *_es(a_gmk), *_es(b0_gkn), *_es(b1_gno), C.c_float(scale),
                                                     int(bool(mask_upper)))
        return c

    def conv2d_fwd(self, inp_nhwc, wei_kyxc, strides=(1, 1), dilations=(1, 1), pads=(0, 0)):
        inp = np.ascontiguousarray(inp_nhwc)
        wei = np.ascontiguousarray(wei_kyxc)
        N, Hi, Wi, Cc = inp.shape
        K, Y, X, _ = wei.shape
        Ho = self.conv_out_len(Hi, Y, strides[0], dilations[0], pads[0], pads[0])
        Wo = self.conv_out_len(Wi, X, strides[1], dilations[1], pads[1], pads[1])
        out = np.zeros((N, Ho, Wo, K), inp.dtype)
        fn = {np.dtype(np.float32): self.lib.ckref_conv2d_fwd_f32,
              np.dtype(np.float16): self.lib.ckref_conv2d_fwd_f16,
              np.dtype(np.int8): self.lib.ckref_conv2d_fwd_i8}[inp.dtype]
        fn(_p(inp), _p(wei), _p(out), N, K, Cc, Hi, Wi, Y, X, Ho, Wo, strides[0], strides[1],
           dilations[0], dilations[1], pads[0], pads[1])
        return out

    def convnd_fwd(self, inp, wei, strides, dilations, pads):
        """1, 2 or 3 spatial dimensions, channels-last tensors, symmetric pads."""
        inp = np.ascontiguousarray(inp)
        wei = np.ascontiguousarray(wei)
        nd = inp.ndim - 2
        in_len, filt = list(inp.shape[1:-1]), list(wei.shape[1:-1])
        out_len = [self.conv_out_len(in_len[i], filt[i], strides[i], dilations[i], pads[i], pads[i]) for i in range(nd)]
        N, Cc, K = inp.shape[0], inp.shape[-1], wei.shape[0]
        out = np.zeros((N, *out_len, K), inp.dtype)
        fn = {np.dtype(np.float32): self.lib.ckref_convnd_fwd_f32,
              np.dtype(np.float16): self.lib.ckref_convnd_fwd_f16,
              np.dtype(np.int8): self.lib.ckref_convnd_fwd_i8}[inp.dtype]
        arr = lambda v: (C.c_int * 3)(*([int(x) for x in v] + [0] * (3 - nd)))
        fn(nd, _p(inp), _p(wei), _p(out), N, K, Cc, arr(in_len), arr(filt), arr(out_len), arr(strides),
           arr(dilations), arr(pads))
        return out

    def conv2d_fwd_bias_relu_f16(self, inp_nhwc, wei_kyxc, bias_k, resi_nhwk=None, strides=(1, 1),
                                 dilations=(1, 1), pads=(0, 0)):
        inp = np.ascontiguousarray(inp_nhwc, np.float16)
        wei = np.ascontiguousarray(wei_kyxc, np.float16)
        bias = np.ascontiguousarray(bias_k, np.float16)
        N, Hi, Wi, Cc = inp.shape
        K, Y, X, _ = wei.shape
        Ho = self.conv_out_len(Hi, Y, strides[0], dilations[0], pads[0], pads[0])
        Wo = self.conv_out_len(Wi, X, strides[1], dilations[1], pads[1], pads[1])
        out = np.zeros((N, Ho, Wo, K), np.float16)
        resi = None if resi_nhwk is None else np.ascontiguousarray(resi_nhwk, np.float16)
        self.lib.ckref_conv2d_fwd_bias_relu_f16(_p(inp), _p(wei), _p(bias), _p(resi) if resi is not None else None,
                                                _p(out), N, K, Cc, Hi, Wi, Y, X, Ho, Wo, strides[0], strides[1],
                                                dilations[0], dilations[1], pads[0], pads[1])
        return out

    def gemm_f16_add_relu(self, a_mk, b_kn, d_mn):
        M, K = a_mk.shape
        _, N = b_kn.shape
        d = np.broadcast_to(d_mn, (M, N))
        e = np.zeros((M, N), np.float16)
        self.lib.ckref_gemm_f16_add_relu(_p(a_mk), _p(b_kn), _p(d), _p(e), M, N, K, *_es(a_mk), *_es(b_kn), *_es(d))
        return e

    def gemm_f16_bilinear(self, a_mk, b_kn, d_mn, alpha, beta):
        M, K = a_mk.shape
        _, N = b_kn.shape
        d = np.broadcast_to(d_mn, (M, N))
        e = np.zeros((M, N), np.float16)
        self.lib.ckref_gemm_f16_bilinear(_p(a_mk), _p(b_kn), _p(d), _p(e), M, N, K, *_es(a_mk), *_es(b_kn), *_es(d),
                                         C.c_float(alpha), C.c_float(beta))
        return e

    def gemm_f16_add_add_fastgelu(self, a_mk, b_kn, d0_mn, d1_mn):
        M, K = a_mk.shape
        _, N = b_kn.shape
        d0 = np.broadcast_to(d0_mn, (M, N))
        d1 = np.broadcast_to(d1_mn, (M, N))
        e = np.zeros((M, N), np.float16)
        self.lib.ckref_gemm_f16_add_add_fastgelu(_p(a_mk), _p(b_kn), _p(d0), _p(d1), _p(e), M, N, K, *_es(a_mk),
                                                 *_es(b_kn), *_es(d0), *_es(d1))
        return e

    def fast_gelu(self, x):
        self.lib.ckref_fast_gelu.restype = C.c_float
        return float(self.lib.ckref_fast_gelu(C.c_float(x)))

    def gemm_bf16(self, a_mk, b_kn):
        M, K = a_mk.shape
        _, N = b_kn.shape
        c = np.zeros((M, N), np.uint16)
        self.lib.ckref_gemm_bf16(_p(a_mk), _p(b_kn), _p(c), M, N, K, *_es(a_mk), *_es(b_kn), C.c_long(N), C.c_long(1))
        return c

    def float_to_bf16(self, x):
        self.lib.ckref_float_to_bf16.restype = C.c_uint16
        self.lib.ckref_float_to_bf16.argtypes = [C.c_float]
        return int(self.lib.ckref_float_to_bf16(float(x)))

    def conv_out_len(self, in_len, filt, stride, dil, pl, pr):
        return int(self.lib.ckref_conv_out_len(in_len, filt, stride, dil, pl, pr))

    def magic_params(self, d):
        m, s = C.c_uint32(), C.c_uint32()
        self.lib.ckref_magic_division_params(C.c_uint32(d), C.byref(m), C.byref(s))
        return m.value, s.value

    def magic_divide(self, n, mult, shift):
        return int(self.lib.ckref_magic_division_divide(n, mult, shift))


_ref = None


def load_ref():
    global _ref
    if _ref is None and os.path.exists(_SO):
        try:
            _ref = _Ref(_SO)
        except OSError:
            _ref = None
    return _ref
