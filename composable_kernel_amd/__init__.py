"""MI355X-native MFMA GEMM hot path behind Composable Kernel's device-operator surface.

    csrc/        HIP kernels for gfx950 + the C ABI (include/ckx.h) -> lib/libckx.so
    host/        C++ operator classes, instance factory, ckx_profiler driver
    capi.py      ctypes binding of the C ABI
    device_ops.py  Python mirror of DeviceGemm / DeviceConvFwd / DeviceBatchedGemmGemm
    host_tensor.py seeded generators for synthetic inputs
"""
from . import capi, device_ops, host_tensor  # noqa: F401
from .device_ops import (  # noqa: F401
    PassThrough, Scale, RequantReluRequant, AddRelu, AddReluAdd, Bilinear, AddAddFastGelu, Relu, ActivationMul2Clamp, RowMajor, ColumnMajor, StreamConfig,
    DeviceGemmInt8, DeviceGemmF16, DeviceGemmBF16, DeviceGemmSplitKInt8, DeviceGemmSplitKF16, DeviceBatchedGemmInt8, DeviceBatchedGemmF16, DeviceGemmMultipleDF16, DeviceGemmMultipleDInt8,
    DeviceConv2dFwdInt8, DeviceConv2dFwdMultipleDInt8, DeviceConv2dFwdF16,
    DeviceConvNdFwdInt8, DeviceConvNdFwdF16,
    DeviceConv2dFwdBiasActivationF16, DeviceBatchedGemmGemmF16, DeviceBatchedGemmSoftmaxGemmF16,
)
