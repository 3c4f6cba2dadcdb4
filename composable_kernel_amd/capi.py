"""ctypes binding of libckx.so -- the C ABI declared in include/ckx.h.

The library is loaded from composable_kernel_amd/lib/ (built in-tree by
composable_kernel_amd.build). There is no fallback: if it is missing, loading
raises, and every operator raises with it.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# CKX_LIB_PATH selects another build of the same library (A/B comparisons of tuning variants)
LIB_PATH = os.environ.get("CKX_LIB_PATH") or os.path.join(HERE, "lib", "libckx.so")

OK, UNSUPPORTED, INVALID_VALUE, HIP_ERROR = 0, -1, -2, -3
ROW_MAJOR, COL_MAJOR = 0, 1
EPI_PASSTHROUGH, EPI_REQUANT_CK, EPI_REQUANT_RND = 0, 1, 2
EPI_ADD_RELU, EPI_ADD_RELU_ADD, EPI_CSHUFFLE_ADD_RELU = 3, 4, 5
EPI_MUL2_CLAMP, EPI_RELU_MUL2_CLAMP = 6, 7   # int8, one fp32 requant scale per output column as the D operand
EPI_BILINEAR, EPI_ADD_ADD_FASTGELU = 8, 9    # fp16 GEMM: alpha * acc + beta * d0; fast_gelu(acc + d0 + d1)
(OP_GEMM_I8, OP_GEMM_F16, OP_CONV2D_FWD_I8, OP_CONV2D_FWD_F16, OP_BATCHED_GEMM_GEMM, OP_GEMM_SPLITK, OP_GEMM_BF16,
 OP_BATCHED_GEMM_SOFTMAX_GEMM) = range(8)
INSTANCE_AUTO = -1
STATIC_WORKSPACE_BYTES = 32 * 1024 * 1024   # CKX_STATIC_WORKSPACE_BYTES

# every symbol include/ckx.h declares
SYMBOLS = [
    "ckx_version", "ckx_last_error", "ckx_num_instances", "ckx_instance_name",
    "ckx_gemm_i8_is_supported", "ckx_gemm_i8", "ckx_gemm_i8_workspace_bytes",
    "ckx_gemm_f16_is_supported", "ckx_gemm_f16", "ckx_gemm_f16_workspace_bytes",
    "ckx_gemm_bf16_is_supported", "ckx_gemm_bf16", "ckx_gemm_bf16_workspace_bytes",
    "ckx_batched_gemm_is_supported", "ckx_batched_gemm_i8", "ckx_batched_gemm_f16",
    "ckx_gemm_splitk_workspace_bytes", "ckx_gemm_i8_splitk", "ckx_gemm_f16_splitk", "ckx_gemm_i8_splitk_noalloc",
    "ckx_gemm_f16_multiple_d_is_supported", "ckx_gemm_f16_multiple_d", "ckx_gemm_f16_bilinear", "ckx_conv2d_fwd_bias_activation_f16",
    "ckx_gemm_i8_multiple_d_is_supported", "ckx_gemm_i8_multiple_d", "ckx_conv2d_fwd_i8_multiple_d",
    "ckx_conv2d_fwd_is_supported", "ckx_conv2d_fwd_i8", "ckx_conv2d_fwd_f16", "ckx_conv2d_fwd_workspace_bytes",
    "ckx_convnd_fwd_is_supported", "ckx_convnd_fwd", "ckx_convnd_fwd_workspace_bytes",
    "ckx_batched_gemm_gemm_f16_is_supported", "ckx_batched_gemm_gemm_f16", "ckx_time_launches",
    "ckx_batched_gemm_softmax_gemm_f16_is_supported", "ckx_batched_gemm_softmax_gemm_f16",
    "ckx_gemm_plan", "ckx_conv2d_fwd_plan", "ckx_set_forced_k_runs", "ckx_set_big_tile_waves",
]


class Conv2dDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "N", "K", "C", "Hi", "Wi", "Y", "X", "Ho", "Wo", "stride_h", "stride_w", "dilation_h",
        "dilation_w", "pad_top", "pad_left", "pad_bottom", "pad_right")]


class ConvNdDesc(C.Structure):
    """ckx_convnd_desc: the first ndim entries of every array are used, slowest dimension first."""
    _fields_ = [("ndim", C.c_int32), ("N", C.c_int32), ("K", C.c_int32), ("C", C.c_int32)] + [
        (n, C.c_int32 * 3) for n in ("in_", "filter", "out", "stride", "dilation", "pad_left", "pad_right")]

    @classmethod
    def make(cls, N, K, C_, in_len, filt, out_len, strides, dilations, left_pads, right_pads):
        nd = len(in_len)
        if nd not in (1, 2, 3) or any(len(v) != nd for v in (filt, out_len, strides, dilations, left_pads, right_pads)):
            raise ValueError("1, 2 or 3 spatial dimensions, every vector of that length")
        arr = lambda v: (C.c_int32 * 3)(*([int(x) for x in v] + [0] * (3 - nd)))
        return cls(nd, int(N), int(K), int(C_), arr(in_len), arr(filt), arr(out_len), arr(strides), arr(dilations),
                   arr(left_pads), arr(right_pads))


LAUNCH_FN = C.CFUNCTYPE(C.c_int, C.c_void_p)

_lib = None


class CkxError(RuntimeError):
    def __init__(self, status, msg):
        super().__init__(f"ckx status {status}: {msg}")
        self.status = status


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            f"{LIB_PATH} is missing: build it with `python -m composable_kernel_amd.build` "
            "(there is no CPU fallback)")
    # In a process that also uses torch (tests, bench), torch's bundled HIP runtime must be the
    # one that gets loaded: it shares its SONAME with the system copy libckx.so names.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(LIB_PATH)
    i32, f32, vp, i64 = C.c_int32, C.c_float, C.c_void_p, C.c_int64
    L.ckx_version.restype = C.c_char_p
    L.ckx_last_error.restype = C.c_char_p
    L.ckx_num_instances.argtypes = [C.c_int]
    L.ckx_instance_name.restype = C.c_char_p
    L.ckx_instance_name.argtypes = [C.c_int, C.c_int]
    shape = [i32] * 6 + [C.c_int] * 3
    L.ckx_gemm_i8_is_supported.argtypes = shape + [C.c_int, C.c_int]
    L.ckx_gemm_i8.argtypes = [vp, vp, vp] + shape + [C.c_int, f32, f32, C.c_int, vp, i64, vp]
    for fn in (L.ckx_gemm_i8_workspace_bytes, L.ckx_gemm_f16_workspace_bytes, L.ckx_gemm_bf16_workspace_bytes):
        fn.restype = i64
        fn.argtypes = [i32, i32, i32, C.c_int]
    L.ckx_gemm_f16_is_supported.argtypes = shape + [C.c_int]
    L.ckx_gemm_f16.argtypes = [vp, vp, vp] + shape + [C.c_int, vp, i64, vp]
    L.ckx_gemm_bf16_is_supported.argtypes = shape + [C.c_int]
    L.ckx_gemm_bf16.argtypes = [vp, vp, vp] + shape + [C.c_int, vp, i64, vp]
    bshape = [i32] * 6 + [i64] * 3 + [i32] + [C.c_int] * 3
    L.ckx_batched_gemm_is_supported.argtypes = [C.c_int] + bshape + [C.c_int, C.c_int]
    L.ckx_batched_gemm_i8.argtypes = [vp, vp, vp] + bshape + [C.c_int, f32, f32, C.c_int, vp]
    L.ckx_batched_gemm_f16.argtypes = [vp, vp, vp] + bshape + [C.c_int, vp]
    L.ckx_gemm_splitk_workspace_bytes.restype = i64
    L.ckx_gemm_splitk_workspace_bytes.argtypes = [C.c_int, i32, i32, i32, i32]
    L.ckx_gemm_i8_splitk.argtypes = [vp, vp, vp] + shape + [C.c_int, f32, f32, C.c_int, i32, vp, i64, vp]
    L.ckx_gemm_f16_splitk.argtypes = [vp, vp, vp] + shape + [C.c_int, i32, vp, i64, vp]
    L.ckx_gemm_i8_splitk_noalloc.argtypes = [vp, vp, vp] + shape + [C.c_int, f32, f32, C.c_int, i32, vp]
    md = [i32] * 8 + [C.c_int] * 3
    L.ckx_gemm_f16_multiple_d_is_supported.argtypes = md + [C.c_int, C.c_int]
    L.ckx_gemm_f16_multiple_d.argtypes = [vp] * 5 + md + [C.c_int, C.c_int, vp, i64, vp]
    mdi = [i32] * 7 + [C.c_int] * 3
    L.ckx_gemm_f16_bilinear.argtypes = [vp] * 4 + mdi + [C.c_float, C.c_float, C.c_int, vp, i64, vp]
    L.ckx_gemm_i8_multiple_d_is_supported.argtypes = mdi + [C.c_int, C.c_int]
    L.ckx_gemm_i8_multiple_d.argtypes = [vp] * 4 + mdi + [C.c_int, C.c_int, vp, i64, vp]
    dp = C.POINTER(Conv2dDesc)
    L.ckx_conv2d_fwd_i8_multiple_d.argtypes = [vp] * 4 + [dp, C.c_int, C.c_int, vp, i64, vp]
    L.ckx_conv2d_fwd_bias_activation_f16.argtypes = [vp] * 5 + [dp, C.c_int, C.c_int, vp, i64, vp]
    L.ckx_conv2d_fwd_is_supported.argtypes = [C.c_int, dp, C.c_int, C.c_int]
    L.ckx_conv2d_fwd_i8.argtypes = [vp, vp, vp, dp, C.c_int, f32, f32, C.c_int, vp, i64, vp]
    L.ckx_conv2d_fwd_f16.argtypes = [vp, vp, vp, dp, C.c_int, vp, i64, vp]
    L.ckx_conv2d_fwd_workspace_bytes.restype = i64
    L.ckx_conv2d_fwd_workspace_bytes.argtypes = [C.c_int, dp, C.c_int]
    ndp = C.POINTER(ConvNdDesc)
    L.ckx_convnd_fwd_is_supported.argtypes = [C.c_int, ndp, C.c_int, C.c_int]
    L.ckx_convnd_fwd.argtypes = [C.c_int, vp, vp, vp, ndp, C.c_int, f32, f32, C.c_int, vp, i64, vp]
    L.ckx_convnd_fwd_workspace_bytes.restype = i64
    L.ckx_convnd_fwd_workspace_bytes.argtypes = [C.c_int, ndp, C.c_int]
    gg = [i32] * 9 + [i64] * 4 + [C.c_int]
    L.ckx_batched_gemm_gemm_f16_is_supported.argtypes = gg
    L.ckx_batched_gemm_gemm_f16.argtypes = [vp] * 4 + gg + [vp]
    gsg = [i32] * 9 + [i64] * 4 + [f32, C.c_int, C.c_int]
    L.ckx_batched_gemm_softmax_gemm_f16_is_supported.argtypes = gsg
    L.ckx_batched_gemm_softmax_gemm_f16.argtypes = [vp] * 4 + gsg + [vp]
    L.ckx_time_launches.argtypes = [LAUNCH_FN, vp, C.c_int, C.c_int, vp, C.POINTER(C.c_float)]
    ip = C.POINTER(C.c_int)
    L.ckx_gemm_plan.argtypes = [C.c_int] + shape + [C.c_int, i32, i64, ip, ip]
    L.ckx_conv2d_fwd_plan.argtypes = [C.c_int, dp, C.c_int, i64, ip, ip]
    L.ckx_set_forced_k_runs.argtypes = [C.c_int]
    L.ckx_set_big_tile_waves.argtypes = [C.c_int]
    _lib = L
    return L


def last_error():
    return lib().ckx_last_error().decode()


def check(status):
    if status != OK:
        raise CkxError(status, last_error())


def time_launches(fn, n_warmup, n_repeat, stream):
    """Mean milliseconds of `fn()` (which must enqueue on `stream` and return a ckx status)."""
    ms = C.c_float()
    cb = LAUNCH_FN(lambda _u: int(fn()))
    check(lib().ckx_time_launches(cb, None, int(n_warmup), int(n_repeat), C.c_void_p(stream or 0), C.byref(ms)))
    return float(ms.value)


def gemm_plan(op, M, N, K, sa=None, sb=None, sc=None, a_layout=ROW_MAJOR, b_layout=COL_MAJOR, epilogue=EPI_PASSTHROUGH,
              batch=1, workspace_bytes=0, instance=INSTANCE_AUTO):
    """(instance, K runs) a launch of this GEMM would use (ckx_gemm_plan); strides default to the dense ones."""
    sa = sa if sa is not None else (K if a_layout == ROW_MAJOR else M)
    sb = sb if sb is not None else (K if b_layout == COL_MAJOR else N)
    sc = sc if sc is not None else N
    inst, runs = C.c_int(instance), C.c_int(0)
    check(lib().ckx_gemm_plan(op, M, N, K, sa, sb, sc, a_layout, b_layout, ROW_MAJOR, epilogue, batch, int(workspace_bytes),
                              C.byref(inst), C.byref(runs)))
    return inst.value, runs.value


def conv2d_fwd_plan(op, desc, epilogue=EPI_PASSTHROUGH, workspace_bytes=0, instance=INSTANCE_AUTO):
    inst, runs = C.c_int(instance), C.c_int(0)
    check(lib().ckx_conv2d_fwd_plan(op, C.byref(desc), epilogue, int(workspace_bytes), C.byref(inst), C.byref(runs)))
    return inst.value, runs.value
