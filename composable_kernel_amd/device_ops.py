"""Python mirror of Composable Kernel's device-operator surface over the C ABI.

The product host layer is C++ (host/ckx/device_ops.hpp); this mirror exists so
that tests and the benchmark can drive the same C entry points with the
reference's vocabulary:

    op  = DeviceGemmInt8(...)                      # one instance
    arg = op.MakeArgumentPointer(p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC,
                                 PassThrough(), PassThrough(), RequantReluRequant(0.03, 1))
    if op.IsSupportedArgument(arg):
        ms = op.MakeInvokerPointer().Run(arg, StreamConfig(stream, time_kernel=True))

Names, argument order and error behaviour follow
include/ck/tensor_operation/gpu/device/device_base.hpp:14-57, device_gemm.hpp:24-41,
device_conv_fwd.hpp:18-39 and (for GEMM-GEMM) upstream's
device_batched_gemm_gemm.hpp:15-56. Pointers are device addresses (ints) or
torch CUDA tensors. Nothing here computes: a missing libckx.so raises.
"""
from dataclasses import dataclass
import ctypes as C

from . import capi


# ---------------------------------------------------------------- functors
class PassThrough:
    """element_wise::PassThrough (unary_element_wise_operation.hpp:13-25)"""
    epilogue = capi.EPI_PASSTHROUGH
    scale_gemm = 1.0
    scale_relu = 1.0


class Scale:
    """element_wise::Scale (unary_element_wise_operation.hpp:27-41): y = scale * x"""

    def __init__(self, scale):
        self.scale = float(scale)


class RequantReluRequant:
    """example/14_gemm_xdl_requant_relu_requant/gemm_xdl_requant_relu_requant_int8.cpp:21-39.
    rounded=False is the literal functor (no rounding, truncating cast);
    rounded=True is sat8(rint(sR*relu(sat8(rint(sG*x)))))."""

    def __init__(self, scale_gemm, scale_relu, rounded=False):
        self.scale_gemm = float(scale_gemm)
        self.scale_relu = float(scale_relu)
        self.epilogue = capi.EPI_REQUANT_RND if rounded else capi.EPI_REQUANT_CK


class AddRelu:
    """element_wise::AddRelu (binary_element_wise_operation.hpp:118-146): y = relu(x0 + x1).
    As an OutElementwiseOperation of the conv operators it acts on the fp32 accumulator
    (reference_conv_fwd_bias_activation.hpp:118-120); as the CDE operation of DeviceGemmMultipleD it
    acts on C already rounded to fp16 (example/03_gemm_bias_relu/gemm_bias_relu_xdl_fp16.cpp:31-40)."""
    epilogue = capi.EPI_ADD_RELU
    cde_epilogue = capi.EPI_CSHUFFLE_ADD_RELU


class AddReluAdd:
    """element_wise::AddReluAdd (element_wise_operation.hpp:46-81): y = relu(x0 + x1) + x2 in fp32."""
    epilogue = capi.EPI_ADD_RELU_ADD
    cde_epilogue = capi.EPI_ADD_RELU_ADD


class Bilinear:
    """element_wise::Bilinear (binary_element_wise_operation.hpp:93-116): y = half(alpha * x0 + beta * float(x1)) with
    x0 the fp32 accumulator (example/02_gemm_bilinear/gemm_bilinear_xdl_fp16.cpp:18-36 is the same functor)."""
    cde_epilogue = capi.EPI_BILINEAR

    def __init__(self, alpha, beta):
        self.alpha_ = float(alpha)
        self.beta_ = float(beta)


class AddAddFastGelu:
    """element_wise::AddAddFastGelu (element_wise_operation.hpp:113-140): e = half(fast_gelu(c + d0 + d1)) on the fp32
    accumulator c, fast_gelu(x) = x * (0.5 + 0.5 * (2 / (1 + exp(-u)) - 1)), u = 2x(0.035677 x^2 + 0.797885)."""
    cde_epilogue = capi.EPI_ADD_ADD_FASTGELU


class Relu:
    """element_wise::Relu (unary_element_wise_operation.hpp): y = x > 0 ? x : 0"""


class ActivationMul2Clamp:
    """element_wise::Activation_Mul2_Clamp<Activation> of upstream Composable Kernel
    (ck/tensor_operation/gpu/element/quantization_operation.hpp as shipped with ROCm; newer than the reference
    snapshot): y = int8(clamp(requant_scale * activation(float(x)), -128, 127)) with one requant scale per output
    column / output channel, passed as the D operand. Activation is PassThrough or Relu."""

    def __init__(self, activation=None):
        activation = activation or PassThrough()
        if not isinstance(activation, (PassThrough, Relu)):
            raise TypeError("activation not built")
        self.activation = activation
        self.epilogue = self.cde_epilogue = (capi.EPI_RELU_MUL2_CLAMP if isinstance(activation, Relu)
                                             else capi.EPI_MUL2_CLAMP)


class RowMajor:
    code = capi.ROW_MAJOR


class ColumnMajor:
    code = capi.COL_MAJOR


@dataclass
class StreamConfig:
    """include/ck/stream_config.hpp:9-13"""
    stream_id_: int = 0
    time_kernel_: bool = False
    nrepeat_: int = 10   # kernel_launch.hpp:20-62: 1 warm-up + 10 timed launches
    nwarmup_: int = 1


def _ptr(x):
    if x is None:
        return 0
    if isinstance(x, int):
        return x
    return int(x.data_ptr())


class BaseArgument:
    p_workspace_ = None       # device pointer (int) set through SetWorkSpacePointer
    workspace_bytes_ = 0
    _workspace_owner = None   # keeps a torch tensor alive when one was passed


class BaseInvoker:
    def __init__(self, op):
        self._op = op

    def Run(self, arg, stream_config=None):
        """Launches; returns mean kernel milliseconds if time_kernel_, else 0
        (kernel_launch.hpp:61,67). Unsupported arguments raise, as the reference's
        Invoker::Run throws (device_gemm_xdl_cshuffle.hpp:475-481)."""
        sc = stream_config or StreamConfig()
        if not self._op.IsSupportedArgument(arg):
            raise RuntimeError("wrong! " + self._op.GetTypeString() + " has invalid setting: "
                               + capi.last_error())
        if not sc.time_kernel_:
            capi.check(self._op._launch(arg, sc.stream_id_))
            return 0.0
        return capi.time_launches(lambda: self._op._launch(arg, sc.stream_id_), sc.nwarmup_,
                                  sc.nrepeat_, sc.stream_id_)


class BaseOperator:
    op_family = None

    def __init__(self, instance=capi.INSTANCE_AUTO):
        self.instance = instance

    def IsSupportedArgument(self, arg):
        return self._supported(arg) == capi.OK

    def GetTypeString(self):
        if self.instance == capi.INSTANCE_AUTO:
            return f"ckx<auto:{self.op_family}>"
        return capi.lib().ckx_instance_name(self.op_family, self.instance).decode()

    def GetWorkSpaceSize(self, arg):
        """Bytes of optional device scratch (split-K); 0 for most problems."""
        return 0

    def SetWorkSpacePointer(self, arg, p, nbytes=None):
        """p: device address or torch CUDA tensor of at least GetWorkSpaceSize(arg) bytes."""
        arg._workspace_owner = p
        arg.p_workspace_ = _ptr(p)
        arg.workspace_bytes_ = int(nbytes if nbytes is not None else self.GetWorkSpaceSize(arg))

    def MakeInvokerPointer(self):
        return BaseInvoker(self)

    @classmethod
    def GetInstances(cls):
        """DeviceOperationInstanceFactory<DeviceOp>::GetInstances()
        (library/include/ck/library/tensor_operation_instance/gpu/gemm.hpp:233-379)"""
        n = capi.lib().ckx_num_instances(cls.op_family)
        return [cls(i) for i in range(n)]


# -------------------------------------------------------------------- GEMM
class _GemmArgument(BaseArgument):
    def __init__(self, p_a, p_b, p_c, M, N, K, sa, sb, sc, a_op, b_op, c_op, layouts):
        self.p_a, self.p_b, self.p_c = _ptr(p_a), _ptr(p_b), _ptr(p_c)
        self.M, self.N, self.K = int(M), int(N), int(K)
        self.StrideA, self.StrideB, self.StrideC = int(sa), int(sb), int(sc)
        self.a_op, self.b_op, self.c_op = a_op, b_op, c_op
        self.layouts = layouts


class _DeviceGemm(BaseOperator):
    def __init__(self, instance=capi.INSTANCE_AUTO, ALayout=RowMajor, BLayout=ColumnMajor, CLayout=RowMajor):
        super().__init__(instance)
        self.layouts = (ALayout.code, BLayout.code, CLayout.code)

    def MakeArgumentPointer(self, p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC, a_element_op=None,
                            b_element_op=None, c_element_op=None):
        a_op = a_element_op or PassThrough()
        b_op = b_element_op or PassThrough()
        if not isinstance(a_op, PassThrough) or not isinstance(b_op, PassThrough):
            raise TypeError("A/B element-wise operations other than PassThrough are not built")
        return _GemmArgument(p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC, a_op, b_op,
                             c_element_op or PassThrough(), self.layouts)


class DeviceGemmInt8(_DeviceGemm):
    """DeviceGemm<..., int8_t, int8_t, int8_t, PassThrough, PassThrough, COp>"""
    op_family = capi.OP_GEMM_I8

    def _supported(self, a):
        return capi.lib().ckx_gemm_i8_is_supported(a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                                   *self.layouts, a.c_op.epilogue, self.instance)

    def GetWorkSpaceSize(self, a):
        return int(capi.lib().ckx_gemm_i8_workspace_bytes(a.M, a.N, a.K, self.instance))

    def _launch(self, a, stream):
        return capi.lib().ckx_gemm_i8(a.p_a, a.p_b, a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                      *self.layouts, a.c_op.epilogue, a.c_op.scale_gemm, a.c_op.scale_relu,
                                      self.instance, a.p_workspace_ or 0, a.workspace_bytes_,
                                      C.c_void_p(stream or 0))


class DeviceGemmF16(_DeviceGemm):
    """DeviceGemm<..., half_t, half_t, half_t, PassThrough, PassThrough, PassThrough>"""
    op_family = capi.OP_GEMM_F16

    def _supported(self, a):
        if not isinstance(a.c_op, PassThrough):
            capi.lib().ckx_gemm_f16_is_supported(-1, 0, 0, 0, 0, 0, 0, 0, 0, 0)  # sets an error string
            return capi.UNSUPPORTED
        return capi.lib().ckx_gemm_f16_is_supported(a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                                    *self.layouts, self.instance)

    def GetWorkSpaceSize(self, a):
        return int(capi.lib().ckx_gemm_f16_workspace_bytes(a.M, a.N, a.K, self.instance))

    def _launch(self, a, stream):
        return capi.lib().ckx_gemm_f16(a.p_a, a.p_b, a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                       *self.layouts, self.instance, a.p_workspace_ or 0, a.workspace_bytes_,
                                       C.c_void_p(stream or 0))


class _DeviceGemmSplitK(_DeviceGemm):
    """DeviceGemmSplitK<...> (device_gemm_splitk.hpp:14-39): MakeArgumentPointer takes a trailing KBatch.
    The workspace (GetWorkSpaceSize) is REQUIRED for KBatch > 1."""

    def MakeArgumentPointer(self, p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC, a_element_op=None,
                            b_element_op=None, c_element_op=None, KBatch=1):
        a = super().MakeArgumentPointer(p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC, a_element_op,
                                        b_element_op, c_element_op)
        a.KBatch = int(KBatch)
        return a

    def GetWorkSpaceSize(self, a):
        return int(capi.lib().ckx_gemm_splitk_workspace_bytes(self.op_family, a.M, a.N, a.K, a.KBatch))


class DeviceGemmSplitKInt8(_DeviceGemmSplitK):
    op_family = capi.OP_GEMM_I8

    def _supported(self, a):
        if not 1 <= a.KBatch <= 8 or self.instance >= capi.lib().ckx_num_instances(capi.OP_GEMM_SPLITK):
            capi.lib().ckx_gemm_i8_is_supported(-1, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0)
            return capi.UNSUPPORTED
        return capi.lib().ckx_gemm_i8_is_supported(a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                                   *self.layouts, a.c_op.epilogue, self.instance)

    def _launch(self, a, stream):
        return capi.lib().ckx_gemm_i8_splitk(a.p_a, a.p_b, a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                             *self.layouts, a.c_op.epilogue, a.c_op.scale_gemm, a.c_op.scale_relu,
                                             self.instance, a.KBatch, a.p_workspace_ or 0, a.workspace_bytes_,
                                             C.c_void_p(stream or 0))


class DeviceGemmSplitKF16(_DeviceGemmSplitK):
    op_family = capi.OP_GEMM_F16

    def _supported(self, a):
        if (not 1 <= a.KBatch <= 8 or self.instance >= capi.lib().ckx_num_instances(capi.OP_GEMM_SPLITK)
                or not isinstance(a.c_op, PassThrough)):
            capi.lib().ckx_gemm_f16_is_supported(-1, 0, 0, 0, 0, 0, 0, 0, 0, 0)
            return capi.UNSUPPORTED
        return capi.lib().ckx_gemm_f16_is_supported(a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                                    *self.layouts, self.instance)

    def _launch(self, a, stream):
        return capi.lib().ckx_gemm_f16_splitk(a.p_a, a.p_b, a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                              *self.layouts, self.instance, a.KBatch, a.p_workspace_ or 0,
                                              a.workspace_bytes_, C.c_void_p(stream or 0))


class DeviceGemmBF16(_DeviceGemm):
    """DeviceGemm<..., bhalf_t, bhalf_t, bhalf_t, PassThrough, PassThrough, PassThrough>"""
    op_family = capi.OP_GEMM_BF16

    def _supported(self, a):
        if not isinstance(a.c_op, PassThrough):
            capi.lib().ckx_gemm_bf16_is_supported(-1, 0, 0, 0, 0, 0, 0, 0, 0, 0)
            return capi.UNSUPPORTED
        return capi.lib().ckx_gemm_bf16_is_supported(a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                                     *self.layouts, self.instance)

    def GetWorkSpaceSize(self, a):
        return int(capi.lib().ckx_gemm_bf16_workspace_bytes(a.M, a.N, a.K, self.instance))

    def _launch(self, a, stream):
        return capi.lib().ckx_gemm_bf16(a.p_a, a.p_b, a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                        *self.layouts, self.instance, a.p_workspace_ or 0, a.workspace_bytes_,
                                        C.c_void_p(stream or 0))


class _DeviceBatchedGemm(_DeviceGemm):
    """DeviceBatchedGemm<...> (device_batched_gemm.hpp:24-45): strided batch, element strides."""

    def MakeArgumentPointer(self, p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC, BatchStrideA, BatchStrideB,
                            BatchStrideC, Batch, a_element_op=None, b_element_op=None, c_element_op=None):
        a = super().MakeArgumentPointer(p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC, a_element_op,
                                        b_element_op, c_element_op)
        a.batch = (int(BatchStrideA), int(BatchStrideB), int(BatchStrideC), int(Batch))
        return a

    def _supported(self, a):
        if self.op_family == capi.OP_GEMM_F16 and not isinstance(a.c_op, PassThrough):
            capi.lib().ckx_gemm_f16_is_supported(-1, 0, 0, 0, 0, 0, 0, 0, 0, 0)
            return capi.UNSUPPORTED
        return capi.lib().ckx_batched_gemm_is_supported(self.op_family, a.M, a.N, a.K, a.StrideA, a.StrideB,
                                                        a.StrideC, *a.batch, *self.layouts, a.c_op.epilogue,
                                                        self.instance)

    def _launch(self, a, stream):
        return self._call(a, a.p_a, a.p_b, a.p_c, stream)


class DeviceBatchedGemmInt8(_DeviceBatchedGemm):
    op_family = capi.OP_GEMM_I8

    def _call(self, a, pa, pb, pc, stream):
        return capi.lib().ckx_batched_gemm_i8(pa, pb, pc, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC, *a.batch,
                                              *self.layouts, a.c_op.epilogue, a.c_op.scale_gemm, a.c_op.scale_relu,
                                              self.instance, C.c_void_p(stream or 0))


class DeviceBatchedGemmF16(_DeviceBatchedGemm):
    op_family = capi.OP_GEMM_F16

    def _call(self, a, pa, pb, pc, stream):
        if not isinstance(a.c_op, PassThrough):
            capi.lib().ckx_gemm_f16_is_supported(-1, 0, 0, 0, 0, 0, 0, 0, 0, 0)
            return capi.UNSUPPORTED
        return capi.lib().ckx_batched_gemm_f16(pa, pb, pc, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC, *a.batch,
                                               *self.layouts, self.instance, C.c_void_p(stream or 0))


class DeviceGemmMultipleDF16(BaseOperator):
    """DeviceGemmMultipleD<Row, Col, Row, half_t, half_t, Tuple<half_t[, half_t]>, half_t, PassThrough,
    PassThrough, CDEOp> (device_gemm_multiple_d.hpp:14-55): E = cde_op(A*B, D0[, D1])."""
    op_family = capi.OP_GEMM_F16

    def __init__(self, instance=capi.INSTANCE_AUTO, ALayout=RowMajor, BLayout=ColumnMajor, DELayout=RowMajor):
        super().__init__(instance)
        self.layouts = (ALayout.code, BLayout.code, DELayout.code)

    def MakeArgumentPointer(self, p_a, p_b, p_ds, p_e, M, N, K, StrideA, StrideB, StrideDs, StrideE,
                            a_element_op=None, b_element_op=None, cde_element_op=None):
        if not 1 <= len(p_ds) <= 2 or len(StrideDs) != len(p_ds):
            raise ValueError("one or two D tensors")
        if not isinstance(cde_element_op, (AddRelu, AddReluAdd, Bilinear, AddAddFastGelu)):
            raise TypeError("CDE element-wise operation not built")
        if len(p_ds) != (2 if isinstance(cde_element_op, (AddReluAdd, AddAddFastGelu)) else 1):
            raise ValueError("number of D tensors does not match the CDE element-wise operation")
        a = _GemmArgument(p_a, p_b, p_e, M, N, K, StrideA, StrideB, StrideE, a_element_op or PassThrough(),
                          b_element_op or PassThrough(), cde_element_op, self.layouts)
        a.p_ds = [_ptr(p) for p in p_ds] + [0] * (2 - len(p_ds))
        a.StrideDs = [int(x) for x in StrideDs] + [0] * (2 - len(p_ds))
        return a

    def _supported(self, a):
        return capi.lib().ckx_gemm_f16_multiple_d_is_supported(
            a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideDs[0], a.StrideDs[1], a.StrideC, *self.layouts,
            a.c_op.cde_epilogue, self.instance)

    def GetWorkSpaceSize(self, a):
        return int(capi.lib().ckx_gemm_f16_workspace_bytes(a.M, a.N, a.K, self.instance))

    def _launch(self, a, stream):
        if isinstance(a.c_op, Bilinear):
            return capi.lib().ckx_gemm_f16_bilinear(
                a.p_a, a.p_b, a.p_ds[0], a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideDs[0], a.StrideC,
                *self.layouts, a.c_op.alpha_, a.c_op.beta_, self.instance, a.p_workspace_ or 0, a.workspace_bytes_,
                C.c_void_p(stream or 0))
        return capi.lib().ckx_gemm_f16_multiple_d(
            a.p_a, a.p_b, a.p_ds[0], a.p_ds[1], a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideDs[0],
            a.StrideDs[1], a.StrideC, *self.layouts, a.c_op.cde_epilogue, self.instance, a.p_workspace_ or 0,
            a.workspace_bytes_, C.c_void_p(stream or 0))


class DeviceGemmMultipleDInt8(BaseOperator):
    """DeviceGemmMultipleD<ALayout, BLayout, Row, int8_t, int8_t, Tuple<float>, int8_t, PassThrough, PassThrough,
    Activation_Mul2_Clamp<Act>> (device_gemm_multiple_d.hpp:14-55): E = cde_op(A*B, D0) with D0 one row of N fp32
    requant scales (stride 0: broadcast over the rows), the per-channel int8 requantisation."""
    op_family = capi.OP_GEMM_I8

    def __init__(self, instance=capi.INSTANCE_AUTO, ALayout=RowMajor, BLayout=ColumnMajor, DELayout=RowMajor):
        super().__init__(instance)
        self.layouts = (ALayout.code, BLayout.code, DELayout.code)

    def MakeArgumentPointer(self, p_a, p_b, p_ds, p_e, M, N, K, StrideA, StrideB, StrideDs, StrideE,
                            a_element_op=None, b_element_op=None, cde_element_op=None):
        if len(p_ds) != 1 or len(StrideDs) != 1:
            raise ValueError("one D tensor: the row of requant scales")
        if not isinstance(cde_element_op, ActivationMul2Clamp):
            raise TypeError("CDE element-wise operation not built")
        a = _GemmArgument(p_a, p_b, p_e, M, N, K, StrideA, StrideB, StrideE, a_element_op or PassThrough(),
                          b_element_op or PassThrough(), cde_element_op, self.layouts)
        a.p_ds = [_ptr(p_ds[0])]
        a.StrideDs = [int(StrideDs[0])]
        return a

    def _supported(self, a):
        return capi.lib().ckx_gemm_i8_multiple_d_is_supported(
            a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideDs[0], a.StrideC, *self.layouts, a.c_op.cde_epilogue,
            self.instance)

    def GetWorkSpaceSize(self, a):
        return int(capi.lib().ckx_gemm_i8_workspace_bytes(a.M, a.N, a.K, self.instance))

    def _launch(self, a, stream):
        return capi.lib().ckx_gemm_i8_multiple_d(
            a.p_a, a.p_b, a.p_ds[0], a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideDs[0], a.StrideC,
            *self.layouts, a.c_op.cde_epilogue, self.instance, a.p_workspace_ or 0, a.workspace_bytes_,
            C.c_void_p(stream or 0))


# -------------------------------------------------------------------- conv
class _ConvArgument(BaseArgument):
    def __init__(self, p_in, p_wei, p_out, desc, out_op):
        self.p_in, self.p_wei, self.p_out = _ptr(p_in), _ptr(p_wei), _ptr(p_out)
        self.desc = desc
        self.out_op = out_op


class _DeviceConvFwd(BaseOperator):
    """DeviceConvFwd<InOp, WeiOp, OutOp>, 2-D NHWC / KYXC / NHWK (device_conv_fwd.hpp:18-39)"""

    def MakeArgumentPointer(self, p_in, p_wei, p_out, N, K, C_, input_spatial_lengths,
                            filter_spatial_lengths, output_spatial_lengths, conv_filter_strides,
                            conv_filter_dilations, input_left_pads, input_right_pads, in_element_op=None,
                            wei_element_op=None, out_element_op=None):
        for v in (input_spatial_lengths, filter_spatial_lengths, output_spatial_lengths,
                  conv_filter_strides, conv_filter_dilations, input_left_pads, input_right_pads):
            if len(v) != 2:
                raise ValueError("only NumDimSpatial == 2 is built")
        d = capi.Conv2dDesc(N, K, C_, *input_spatial_lengths, *filter_spatial_lengths,
                            *output_spatial_lengths, *conv_filter_strides, *conv_filter_dilations,
                            *input_left_pads, *input_right_pads)
        return _ConvArgument(p_in, p_wei, p_out, d, out_element_op or PassThrough())

    def _supported(self, a):
        return capi.lib().ckx_conv2d_fwd_is_supported(self.op_family, C.byref(a.desc), a.out_op.epilogue,
                                                      self.instance)

    def GetWorkSpaceSize(self, a):
        return int(capi.lib().ckx_conv2d_fwd_workspace_bytes(self.op_family, C.byref(a.desc), self.instance))


class DeviceConv2dFwdInt8(_DeviceConvFwd):
    op_family = capi.OP_CONV2D_FWD_I8

    def _launch(self, a, stream):
        return capi.lib().ckx_conv2d_fwd_i8(a.p_in, a.p_wei, a.p_out, C.byref(a.desc), a.out_op.epilogue,
                                            a.out_op.scale_gemm, a.out_op.scale_relu, self.instance,
                                            a.p_workspace_ or 0, a.workspace_bytes_, C.c_void_p(stream or 0))


class DeviceConv2dFwdMultipleDInt8(_DeviceConvFwd):
    """2-D conv forward, int8, with one fp32 requant scale per output channel as the D operand and
    Activation_Mul2_Clamp<Act> as the output operation (upstream's per-channel conv quantisation; the
    DeviceConvFwd argument list of device_conv_fwd.hpp:18-39 with the scale pointer after p_out)."""
    op_family = capi.OP_CONV2D_FWD_I8

    def MakeArgumentPointer(self, p_in, p_wei, p_out, p_scale, *rest):
        if not isinstance(rest[-1], ActivationMul2Clamp):
            raise TypeError("output operation not built")
        a = super().MakeArgumentPointer(p_in, p_wei, p_out, *rest)
        a.p_scale = _ptr(p_scale)
        return a

    def _launch(self, a, stream):
        return capi.lib().ckx_conv2d_fwd_i8_multiple_d(a.p_in, a.p_wei, a.p_scale, a.p_out, C.byref(a.desc),
                                                       a.out_op.epilogue, self.instance, a.p_workspace_ or 0,
                                                       a.workspace_bytes_, C.c_void_p(stream or 0))


class DeviceConv2dFwdF16(_DeviceConvFwd):
    op_family = capi.OP_CONV2D_FWD_F16

    def _launch(self, a, stream):
        return capi.lib().ckx_conv2d_fwd_f16(a.p_in, a.p_wei, a.p_out, C.byref(a.desc), self.instance,
                                             a.p_workspace_ or 0, a.workspace_bytes_, C.c_void_p(stream or 0))


class _DeviceConvNdFwd(BaseOperator):
    """DeviceConvFwd<InOp, WeiOp, OutOp> as implemented by DeviceConvNDFwdXdl_Input_N_Hi_Wi_C_Weight_K_Y_X_C_
    Output_N_Ho_Wo_K<..., NumDimSpatial> (device_convnd_fwd_xdl_nhwc_kyxc_nhwk.hpp:76-1046): NWC / NHWC / NDHWC
    input, KXC / KYXC / KZYXC weight, NWK / NHWK / NDHWK output; every vector has NumDimSpatial entries."""

    def __init__(self, NumDimSpatial=2, instance=capi.INSTANCE_AUTO):
        super().__init__(instance)
        if NumDimSpatial not in (1, 2, 3):
            raise ValueError("NumDimSpatial is 1, 2 or 3")
        self.NumDimSpatial = NumDimSpatial

    def MakeArgumentPointer(self, p_in, p_wei, p_out, N, K, C_, input_spatial_lengths,
                            filter_spatial_lengths, output_spatial_lengths, conv_filter_strides,
                            conv_filter_dilations, input_left_pads, input_right_pads, in_element_op=None,
                            wei_element_op=None, out_element_op=None):
        if len(input_spatial_lengths) != self.NumDimSpatial:
            raise ValueError(f"this operator has NumDimSpatial == {self.NumDimSpatial}")
        d = capi.ConvNdDesc.make(N, K, C_, input_spatial_lengths, filter_spatial_lengths, output_spatial_lengths,
                                 conv_filter_strides, conv_filter_dilations, input_left_pads, input_right_pads)
        return _ConvArgument(p_in, p_wei, p_out, d, out_element_op or PassThrough())

    def _supported(self, a):
        return capi.lib().ckx_convnd_fwd_is_supported(self.op_family, C.byref(a.desc), a.out_op.epilogue, self.instance)

    def GetWorkSpaceSize(self, a):
        return int(capi.lib().ckx_convnd_fwd_workspace_bytes(self.op_family, C.byref(a.desc), self.instance))

    def _launch(self, a, stream):
        sg = getattr(a.out_op, "scale_gemm", 1.0)
        sr = getattr(a.out_op, "scale_relu", 1.0)
        return capi.lib().ckx_convnd_fwd(self.op_family, a.p_in, a.p_wei, a.p_out, C.byref(a.desc), a.out_op.epilogue,
                                         sg, sr, self.instance, a.p_workspace_ or 0, a.workspace_bytes_,
                                         C.c_void_p(stream or 0))


    @classmethod
    def GetInstances(cls, NumDimSpatial=2):
        """ConvolutionFwdInstances<T, T, T>::Get<NumDimSpatial>() (library/include/ck/library/utility/conv_util.hpp:288-397)"""
        return [cls(NumDimSpatial, i) for i in range(capi.lib().ckx_num_instances(cls.op_family))]


class DeviceConvNdFwdInt8(_DeviceConvNdFwd):
    op_family = capi.OP_CONV2D_FWD_I8


class DeviceConvNdFwdF16(_DeviceConvNdFwd):
    op_family = capi.OP_CONV2D_FWD_F16


class DeviceConv2dFwdBiasActivationF16(_DeviceConvFwd):
    """DeviceConvFwdBiasActivation<InOp, WeiOp, AddRelu> and DeviceConvFwdBiasActivationAdd<..., AddReluAdd>
    (device_conv_fwd_bias_activation.hpp:18-41, device_conv_fwd_bias_activation_add.hpp): p_bias is a
    [K] vector; p_resi (NHWK, like the output) is given for the Add form only."""
    op_family = capi.OP_CONV2D_FWD_F16

    def MakeArgumentPointer(self, p_in, p_wei, p_out, p_bias, *rest):
        # (p_resi,) N, K, C, spatial vectors..., element-wise operations: the Add form has one more pointer
        p_resi = None
        if len(rest) == 14:
            p_resi, rest = rest[0], rest[1:]
        if len(rest) != 13:
            raise TypeError("expected N, K, C, 7 vectors and 3 element-wise operations")
        a = super().MakeArgumentPointer(p_in, p_wei, p_out, *rest)
        if not isinstance(a.out_op, (AddRelu, AddReluAdd)) or isinstance(a.out_op, AddReluAdd) != (p_resi is not None):
            raise TypeError("out_element_op must be AddRelu (no residual) or AddReluAdd (with residual)")
        a.p_bias, a.p_resi = _ptr(p_bias), _ptr(p_resi)
        return a

    def _launch(self, a, stream):
        return capi.lib().ckx_conv2d_fwd_bias_activation_f16(
            a.p_in, a.p_wei, a.p_out, a.p_bias, a.p_resi, C.byref(a.desc), a.out_op.epilogue, self.instance,
            a.p_workspace_ or 0, a.workspace_bytes_, C.c_void_p(stream or 0))


# --------------------------------------------------------------- GEMM-GEMM
class _GemmGemmArgument(BaseArgument):
    pass


class DeviceBatchedGemmGemmF16(BaseOperator):
    """DeviceBatchedGemmGemm<Row, Col, Row, Row, half x4, PassThrough x5>"""
    op_family = capi.OP_BATCHED_GEMM_GEMM

    def MakeArgumentPointer(self, p_a, p_b0, p_b1, p_c, M, N, K, O, Batch, StrideA, StrideB0, StrideB1,
                            StrideC, BatchStrideA, BatchStrideB0, BatchStrideB1, BatchStrideC,
                            a_element_op=None, b0_element_op=None, acc0_element_op=None,
                            b1_element_op=None, c_element_op=None):
        for op in (a_element_op, b0_element_op, acc0_element_op, b1_element_op, c_element_op):
            if op is not None and not isinstance(op, PassThrough):
                raise TypeError("only PassThrough element-wise operations are built")
        a = _GemmGemmArgument()
        a.ptrs = (_ptr(p_a), _ptr(p_b0), _ptr(p_b1), _ptr(p_c))
        a.dims = (int(M), int(N), int(K), int(O), int(Batch), int(StrideA), int(StrideB0), int(StrideB1),
                  int(StrideC), int(BatchStrideA), int(BatchStrideB0), int(BatchStrideB1), int(BatchStrideC))
        return a

    def _supported(self, a):
        return capi.lib().ckx_batched_gemm_gemm_f16_is_supported(*a.dims, self.instance)

    def _launch(self, a, stream):
        return capi.lib().ckx_batched_gemm_gemm_f16(*a.ptrs, *a.dims, self.instance, C.c_void_p(stream or 0))


class DeviceBatchedGemmSoftmaxGemmF16(BaseOperator):
    """DeviceBatchedGemmSoftmaxGemm<Row, Col, Row, Row, half x4, PassThrough, PassThrough, Scale, PassThrough,
    PassThrough, MaskOutUpperTriangle> (upstream's device_batched_gemm_softmax_gemm.hpp:29-62):
    C[g] = half(half(softmax_n(mask(scale * A[g] B0[g]))) B1[g])."""
    op_family = capi.OP_BATCHED_GEMM_SOFTMAX_GEMM

    def __init__(self, instance=capi.INSTANCE_AUTO, MaskOutUpperTriangle=False):
        super().__init__(instance)
        self.mask = bool(MaskOutUpperTriangle)

    def MakeArgumentPointer(self, p_a, p_b0, p_b1, p_c, M, N, K, O, Batch, StrideA, StrideB0, StrideB1,
                            StrideC, BatchStrideA, BatchStrideB0, BatchStrideB1, BatchStrideC,
                            a_element_op=None, b0_element_op=None, acc0_element_op=None,
                            b1_element_op=None, c_element_op=None):
        for op in (a_element_op, b0_element_op, b1_element_op, c_element_op):
            if op is not None and not isinstance(op, PassThrough):
                raise TypeError("only PassThrough element-wise operations are built for A, B0, B1 and C")
        if acc0_element_op is not None and not isinstance(acc0_element_op, (Scale, PassThrough)):
            raise TypeError("the score operation is Scale or PassThrough")
        a = _GemmGemmArgument()
        a.ptrs = (_ptr(p_a), _ptr(p_b0), _ptr(p_b1), _ptr(p_c))
        a.dims = (int(M), int(N), int(K), int(O), int(Batch), int(StrideA), int(StrideB0), int(StrideB1),
                  int(StrideC), int(BatchStrideA), int(BatchStrideB0), int(BatchStrideB1), int(BatchStrideC))
        a.scale = acc0_element_op.scale if isinstance(acc0_element_op, Scale) else 1.0
        return a

    def _supported(self, a):
        return capi.lib().ckx_batched_gemm_softmax_gemm_f16_is_supported(*a.dims, a.scale, int(self.mask), self.instance)

    def _launch(self, a, stream):
        return capi.lib().ckx_batched_gemm_softmax_gemm_f16(*a.ptrs, *a.dims, a.scale, int(self.mask), self.instance,
                                                            C.c_void_p(stream or 0))
