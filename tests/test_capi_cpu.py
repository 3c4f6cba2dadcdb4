"""CPU-only checks of the drop-in boundary: the C-ABI library loads, exports every symbol
include/ckx.h declares, and its pure-host argument validation behaves like the reference's
IsSupportedArgument (no kernel is launched here)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import splitmix64, uniform_f16, uniform_int8

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "ckx.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(ckx_[a-z0-9_]+)\s*\(", hdr)) - {"ckx_launch_fn"}
    assert declared == set(capi.SYMBOLS)
    L = capi.lib()
    for name in sorted(declared):
        assert getattr(L, name) is not None
    assert b"gfx950" in L.ckx_version()


def test_instance_factory_lists_named_instances():
    L = capi.lib()
    for op in range(5):
        n = L.ckx_num_instances(op)
        assert n >= 1
        names = [L.ckx_instance_name(op, i).decode() for i in range(n)]
        assert len(set(names)) == n
        assert L.ckx_instance_name(op, n) is None
    assert L.ckx_num_instances(99) == 0
    assert len(ck.DeviceGemmInt8.GetInstances()) == L.ckx_num_instances(capi.OP_GEMM_I8)


def test_gemm_argument_validation_is_pure_host_logic():
    op = ck.DeviceGemmInt8()
    ok = op.MakeArgumentPointer(0, 0, 0, 1024, 1024, 1024, 1024, 1024, 1024, None, None,
                                ck.RequantReluRequant(0.5, 0.03, rounded=True))
    assert op.IsSupportedArgument(ok)
    # stride below K; column-major C; >= 2 GiB operand
    for bad in [
        op.MakeArgumentPointer(0, 0, 0, 64, 64, 128, 64, 128, 64),
        op.MakeArgumentPointer(0, 0, 0, 1 << 16, 64, 1 << 15, 1 << 15, 1 << 15, 64),
    ]:
        assert not op.IsSupportedArgument(bad)
        assert capi.last_error()
    assert not ck.DeviceGemmInt8(CLayout=ck.ColumnMajor).IsSupportedArgument(ok)
    assert not ck.DeviceGemmInt8(instance=999).IsSupportedArgument(ok)
    f16 = ck.DeviceGemmF16()
    assert f16.IsSupportedArgument(f16.MakeArgumentPointer(0, 0, 0, 4096, 4096, 4096, 4096, 4096, 4096))
    # K not a multiple of 16 bytes (the reference's KPadding / MNKPadding instances): the vectorised instances
    # refuse, the element-wise instance -- the last of the list -- and the automatic choice accept
    last = capi.lib().ckx_num_instances(capi.OP_GEMM_I8) - 1
    assert b"Generic" in capi.lib().ckx_instance_name(capi.OP_GEMM_I8, last)
    for cls, (M, N, K) in ((ck.DeviceGemmInt8, (64, 64, 100)), (ck.DeviceGemmF16, (64, 64, 60))):
        assert cls().IsSupportedArgument(cls().MakeArgumentPointer(0, 0, 0, M, N, K, K, K, N))
        assert cls(last).IsSupportedArgument(cls(last).MakeArgumentPointer(0, 0, 0, M, N, K, K, K, N))
        for inst in range(last):
            assert not cls(inst).IsSupportedArgument(cls(inst).MakeArgumentPointer(0, 0, 0, 16, N, K, K, K, N))
    # a functor the fp16 operator does not fuse
    assert not f16.IsSupportedArgument(
        f16.MakeArgumentPointer(0, 0, 0, 64, 64, 64, 64, 64, 64, None, None, ck.RequantReluRequant(1, 1)))
    with pytest.raises(RuntimeError):
        op.MakeInvokerPointer().Run(op.MakeArgumentPointer(0, 0, 0, 64, 64, 128, 64, 128, 64))


def test_conv_argument_validation():
    op = ck.DeviceConv2dFwdF16()
    mk = lambda C_, osp: op.MakeArgumentPointer(0, 0, 0, 256, 64, C_, [56, 56], [3, 3], osp, [1, 1], [1, 1],
                                                [1, 1], [1, 1])
    assert op.IsSupportedArgument(mk(64, [56, 56]))
    # C * 2 bytes not a multiple of 16 (ConvolutionForwardSpecialization::OddC): element-wise instance and AUTO only
    assert op.IsSupportedArgument(mk(3, [56, 56]))
    n = capi.lib().ckx_num_instances(capi.OP_CONV2D_FWD_F16)
    assert ck.DeviceConv2dFwdF16(n - 1).IsSupportedArgument(mk(3, [56, 56]))
    assert not any(ck.DeviceConv2dFwdF16(i).IsSupportedArgument(mk(3, [56, 56])) for i in range(n - 1))
    assert not op.IsSupportedArgument(mk(64, [55, 56]))     # output size does not follow from the geometry
    with pytest.raises(ValueError):
        op.MakeArgumentPointer(0, 0, 0, 1, 1, 8, [8], [3], [6], [1], [1], [0], [0])   # only 2-D is built


def test_gemm_gemm_argument_validation():
    op = ck.DeviceBatchedGemmGemmF16()
    mk = lambda K, O: op.MakeArgumentPointer(0, 0, 0, 0, 512, 512, K, O, 64, K, K, O, O, 512 * K, 512 * K,
                                             512 * O, 512 * O)
    assert op.IsSupportedArgument(mk(64, 64))
    assert op.IsSupportedArgument(mk(128, 128))
    assert not op.IsSupportedArgument(mk(256, 64))
    assert not op.IsSupportedArgument(mk(60, 64))
    # B0 / B1 of one batch are addressed through 32-bit offsets: 70000 rows of 16384 elements are 2.3 GB
    wide = lambda sb0, sb1: op.MakeArgumentPointer(0, 0, 0, 0, 128, 70000, 64, 64, 1, 64, sb0, sb1, 64, 0, 0, 0, 0)
    assert op.IsSupportedArgument(wide(64, 64))
    assert not op.IsSupportedArgument(wide(16384, 64))
    assert not op.IsSupportedArgument(wide(64, 16384))
    assert "2 GiB" in capi.last_error()


def test_generators_are_counter_based_and_in_range():
    # first two outputs of the published splitmix64 generator for seed 1234567
    z = splitmix64(1234567, 2)
    assert [int(v) for v in z] == [6457827717110365317, 3203168211198807973]
    a = uniform_int8((1000,), -5, 5, 7)
    assert a.min() == -5 and a.max() == 5
    np.testing.assert_array_equal(uniform_int8((1000,), -5, 5, 7)[:100], uniform_int8((100,), -5, 5, 7))
    h = uniform_f16((4096,), -1, 1, 9)
    assert h.dtype == np.float16 and -1 <= h.min() and h.max() <= 1 and abs(float(h.astype(np.float32).mean())) < 0.05


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", str(tmp_path / "libckx.so"))
    with pytest.raises(FileNotFoundError):
        capi.lib()


def test_build_guards_for_the_hand_waited_kernels():
    """The build reads every kernel's register report and refuses vector register spills in the kernels whose LDS
    fragment reads are waited for by hand; it knows which compiler those kernels were validated with."""
    from composable_kernel_amd import build
    report = """
gemm_tile.hpp:1172:1: remark: Function Name: _ZN3ckx16gemm_tile_kernelILi0ELi256ELi256EEvNS_8GemmArgsE [-Rpass-analysis=kernel-resource-usage]
gemm_tile.hpp:1172:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]
gemm_tile.hpp:1172:1: remark:     VGPRs Spill: 7 [-Rpass-analysis=kernel-resource-usage]
gemm_gemm.hpp:400:1: remark: Function Name: _ZN3ckx16gemm_gemm_kernelILi4EEEvNS_12GemmGemmArgsE [-Rpass-analysis=kernel-resource-usage]
gemm_gemm.hpp:400:1: remark:     VGPRs Spill: 4 [-Rpass-analysis=kernel-resource-usage]
conv_patch.hpp:410:1: remark: Function Name: _ZN3ckx17conv_patch_kernelILi1EEEvNS_13ConvPatchArgsE [-Rpass-analysis=kernel-resource-usage]
conv_patch.hpp:410:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
"""
    assert build.vgpr_spills(report) == [("_ZN3ckx16gemm_tile_kernelILi0ELi256ELi256EEvNS_8GemmArgsE", 7)]
    # ... and scratch memory of any origin in them (a per-lane array that did not stay in registers counts like a spill)
    private_array = """
gemm_tile.hpp:1500:1: remark: Function Name: _ZN3ckx16gemm_tile_kernelILi1ELi256ELi64ELi8ELi1ELi128ELi2ELi2ELb0ELb0ELb0EEEvNS_8GemmArgsE [-Rpass-analysis=kernel-resource-usage]
gemm_tile.hpp:1500:1: remark:     ScratchSize [bytes/lane]: 40 [-Rpass-analysis=kernel-resource-usage]
gemm_tile.hpp:1500:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
gemm_gemm.hpp:400:1: remark: Function Name: _ZN3ckx16gemm_gemm_kernelILi4EEEvNS_12GemmGemmArgsE [-Rpass-analysis=kernel-resource-usage]
gemm_gemm.hpp:400:1: remark:     ScratchSize [bytes/lane]: 16 [-Rpass-analysis=kernel-resource-usage]
"""
    assert build.vgpr_spills(private_array) == []
    assert build.scratch_users(private_array) == [
        ("_ZN3ckx16gemm_tile_kernelILi1ELi256ELi64ELi8ELi1ELi128ELi2ELi2ELb0ELb0ELb0EEEvNS_8GemmArgsE", 40)]
    # the input-patch conv kernel keeps its weights, and nothing else, in AccVGPRs, and has no scratch
    patch = """
conv_patch.hpp:500:1: remark: Function Name: _ZN3ckx17conv_patch_kernelILi1ELi7ELb0EEEvNS_13ConvPatchArgsE [-Rpass-analysis=kernel-resource-usage]
conv_patch.hpp:500:1: remark:     AGPRs: 144 [-Rpass-analysis=kernel-resource-usage]
conv_patch.hpp:500:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
conv_patch.hpp:500:1: remark: Function Name: _ZN3ckx17conv_patch_kernelILi0ELi7ELb0EEEvNS_13ConvPatchArgsE [-Rpass-analysis=kernel-resource-usage]
conv_patch.hpp:500:1: remark:     AGPRs: 200 [-Rpass-analysis=kernel-resource-usage]
conv_patch.hpp:500:1: remark:     ScratchSize [bytes/lane]: 16 [-Rpass-analysis=kernel-resource-usage]
"""
    assert build.patch_register_faults(patch) == [
        ("_ZN3ckx17conv_patch_kernelILi0ELi7ELb0EEEvNS_13ConvPatchArgsE", "200 AccVGPRs"),
        ("_ZN3ckx17conv_patch_kernelILi0ELi7ELb0EEEvNS_13ConvPatchArgsE", "16 bytes of scratch per lane")]
    # ... and its 128-channel form: 60 of the 72 fp16 fragments (240 AccVGPRs), all 36 int8 ones (144)
    wide = """
conv_patch_wide.hpp:390:1: remark: Function Name: _ZN3ckx22conv_patch_wide_kernelILi1ELb0EEEvNS_13ConvPatchArgsE [-Rpass-analysis=kernel-resource-usage]
conv_patch_wide.hpp:390:1: remark:     AGPRs: 240 [-Rpass-analysis=kernel-resource-usage]
conv_patch_wide.hpp:390:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
conv_patch_wide.hpp:390:1: remark: Function Name: _ZN3ckx22conv_patch_wide_kernelILi0ELb0EEEvNS_13ConvPatchArgsE [-Rpass-analysis=kernel-resource-usage]
conv_patch_wide.hpp:390:1: remark:     AGPRs: 128 [-Rpass-analysis=kernel-resource-usage]
conv_patch_wide.hpp:390:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
"""
    assert build.patch_register_faults(wide) == [("_ZN3ckx22conv_patch_wide_kernelILi0ELb0EEEvNS_13ConvPatchArgsE", "128 AccVGPRs")]
    assert "-Rpass-analysis=kernel-resource-usage" in build.DEVICE_FLAGS
    assert "clang version" in build.compiler_version()
    assert all("clang version" in v for v in build.VALIDATED_COMPILERS)


def test_d_operand_epilogues_with_k_major_operands_run_on_auto_or_the_element_granular_instance_only():
    """The is_supported answers per instance and layout, as include/ckx.h states them: with A column-major or B
    row-major the D-operand epilogues (per-column requant scales, the fp16 add / scale / GELU functors) are
    supported by CKX_INSTANCE_AUTO and by the element-granular instance (the last of the family) and by no explicit
    tile or skinny instance; with A row-major and B column-major every instance that takes the shape supports them."""
    L = capi.lib()
    M, N, K = 16, 256, 512   # (16 rows: within the reach of every skinny instance)
    n_i8, n_f16 = L.ckx_num_instances(capi.OP_GEMM_I8), L.ckx_num_instances(capi.OP_GEMM_F16)
    lay = {"mk_nk": (capi.ROW_MAJOR, capi.COL_MAJOR), "km_nk": (capi.COL_MAJOR, capi.COL_MAJOR),
           "mk_kn": (capi.ROW_MAJOR, capi.ROW_MAJOR), "km_kn": (capi.COL_MAJOR, capi.ROW_MAJOR)}
    for name, (al, bl) in lay.items():
        sa, sb = (K if al == capi.ROW_MAJOR else M), (K if bl == capi.COL_MAJOR else N)
        for inst in [capi.INSTANCE_AUTO] + list(range(n_i8)):
            st = L.ckx_gemm_i8_multiple_d_is_supported(M, N, K, sa, sb, 0, N, al, bl, capi.ROW_MAJOR, capi.EPI_MUL2_CLAMP, inst)
            if name == "mk_nk" or inst in (capi.INSTANCE_AUTO, n_i8 - 1):
                assert st == capi.OK, (name, inst, capi.last_error())
            else:
                assert st == capi.UNSUPPORTED, (name, inst)
        for inst in [capi.INSTANCE_AUTO] + list(range(n_f16)):
            st = L.ckx_gemm_f16_multiple_d_is_supported(M, N, K, sa, sb, 0, N, N, al, bl, capi.ROW_MAJOR,
                                                        capi.EPI_ADD_ADD_FASTGELU, inst)
            if name == "mk_nk" or inst in (capi.INSTANCE_AUTO, n_f16 - 1):
                assert st == capi.OK, (name, inst, capi.last_error())
            else:
                assert st == capi.UNSUPPORTED, (name, inst)
