"""GPU parity of the GEMM layouts with a K-major operand through the C ABI: A column-major ("km") and / or
B row-major ("kn"), C row-major -- the km_kn, km_nk and mk_kn instance lists of the reference
(test/gemm/gemm_int8.cpp, gemm_fp16.cpp and gemm_bf16.cpp run all four A/B layout combinations;
library/src/tensor_operation_instance/gpu/gemm/device_gemm_xdl_*_{km_kn,km_nk,mk_kn}_mn_instance.cpp).
int8 is bit-exact; fp16 / bf16 within rtol = atol = 1e-2. The oracle gets the same arrays as strided
[M,K] / [K,N] views, so a transposed or shifted operand in the kernel cannot cancel out."""
import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_bf16, uniform_f16, uniform_int8
from oracle import fast, lit

pytestmark = pytest.mark.gpu

LAYOUTS = {          # name -> (A layout, B layout)
    "km_kn": (ck.ColumnMajor, ck.RowMajor),
    "km_nk": (ck.ColumnMajor, ck.ColumnMajor),
    "mk_kn": (ck.RowMajor, ck.RowMajor),
}
TILES = [0, 1, 2, 3, 4, 7, 8]     # tile instances of 64 rows and more


def _operands(kind, layout, M, N, K, seed, pad_a=0, pad_b=0):
    """Host arrays as stored (with `pad` extra elements per stored row) and their logical [M,K] / [K,N] views."""
    gen = {"i8": lambda s, sd: uniform_int8(s, -8, 8, sd), "f16": lambda s, sd: uniform_f16(s, -1, 1, sd),
           "bf16": lambda s, sd: uniform_bf16(s, -1, 1, sd)}[kind]
    al, bl = LAYOUTS[layout]
    if al is ck.ColumnMajor:
        a_st = gen((K, M + pad_a), seed)
        a_mk = a_st[:, :M].T
    else:
        a_st = gen((M, K + pad_a), seed)
        a_mk = a_st[:, :K]
    if bl is ck.RowMajor:
        b_st = gen((K, N + pad_b), seed + 1)
        b_kn = b_st[:, :N]
    else:
        b_st = gen((N, K + pad_b), seed + 1)
        b_kn = b_st[:, :K].T
    return a_st, b_st, a_mk, b_kn


def _run(kind, layout, a_st, b_st, M, N, K, instance=capi.INSTANCE_AUTO, c_op=None, workspace=False, k_batch=0,
         expect_unsupported=False):
    import torch
    import gpu_util
    al, bl = LAYOUTS[layout]
    tdt = torch.int8 if kind == "i8" else torch.int16
    raw = (lambda x: x) if kind == "i8" else (lambda x: x.view(np.int16))
    da, db = torch.from_numpy(raw(np.ascontiguousarray(a_st))).cuda(), torch.from_numpy(raw(np.ascontiguousarray(b_st))).cuda()
    dc = torch.full((M, N), 77 if kind == "i8" else 0x7E00, dtype=tdt, device="cuda")   # 0x7E00: fp16 NaN
    if k_batch:
        cls = {"i8": ck.DeviceGemmSplitKInt8, "f16": ck.DeviceGemmSplitKF16}[kind]
    else:
        cls = {"i8": ck.DeviceGemmInt8, "f16": ck.DeviceGemmF16, "bf16": ck.DeviceGemmBF16}[kind]
    op = cls(instance, ALayout=al, BLayout=bl)
    args = [da, db, dc, M, N, K, a_st.shape[1], b_st.shape[1], N, None, None, c_op]
    if k_batch:
        args.append(k_batch)
    arg = op.MakeArgumentPointer(*args)
    if expect_unsupported:
        assert not op.IsSupportedArgument(arg)
        with pytest.raises(RuntimeError):
            op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
        return None
    assert op.IsSupportedArgument(arg), capi.last_error()
    if workspace or k_batch:
        ws = torch.full((max(op.GetWorkSpaceSize(arg), 16),), 0x7F, dtype=torch.uint8, device="cuda")
        op.SetWorkSpacePointer(arg, ws)
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    out = dc.cpu().numpy()
    return out if kind == "i8" else out.view(np.float16 if kind == "f16" else np.uint16)


def _check(kind, out, a_mk, b_kn, c_op=None, big=False):
    if kind == "i8":
        epi = (lit.EPI_REQUANT_RND, c_op.scale_gemm, c_op.scale_relu) if c_op else (lit.EPI_PASSTHROUGH, 1.0, 1.0)
        ref = (fast if big else lit).gemm_i8(a_mk, b_kn, *epi)
        np.testing.assert_array_equal(out, ref)
    elif kind == "f16":
        ref = (fast if big else lit).gemm_f16(a_mk, b_kn)
        bad, max_err = lit.check_err_f16(out, ref, 1e-2, 1e-2)
        assert bad == 0, f"{bad} outside tolerance, max err {max_err}"
    else:
        ref = (fast if big else lit).gemm_bf16(a_mk, b_kn)
        o, r = fast.bf16_to_f32(out), fast.bf16_to_f32(ref)
        assert np.all(np.isfinite(o))
        assert np.all(np.abs(o - r) <= 1e-2 + 1e-2 * np.abs(r)), np.abs(o - r).max()


# M, N multiples of 16 (the contiguous extent of a K-major operand must be whole 16-byte vectors, also for int8)
SHAPES = [(256, 256, 256), (304, 208, 192), (16, 144, 1040), (528, 80, 2048), (64, 64, 64), (272, 400, 96)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO] + TILES)
@pytest.mark.parametrize("layout", sorted(LAYOUTS))
def test_int8_requant_gemm_layouts_bit_exact(layout, instance, shape):
    M, N, K = shape
    a_st, b_st, a_mk, b_kn = _operands("i8", layout, M, N, K, 1000 + M)
    c_op = ck.RequantReluRequant(0.03, 0.6, rounded=True)
    _check("i8", _run("i8", layout, a_st, b_st, M, N, K, instance, c_op), a_mk, b_kn, c_op)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 0, 2, 4, 8])
@pytest.mark.parametrize("layout", sorted(LAYOUTS))
@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_fp16_bf16_gemm_layouts(kind, layout, instance, shape):
    M, N, K = shape
    a_st, b_st, a_mk, b_kn = _operands(kind, layout, M, N, K, 1100 + N)
    _check(kind, _run(kind, layout, a_st, b_st, M, N, K, instance), a_mk, b_kn)


@pytest.mark.parametrize("layout", sorted(LAYOUTS))
@pytest.mark.parametrize("kind", ["i8", "f16"])
def test_layouts_padded_strides_and_k_tails(kind, layout):
    """Strides larger than the contiguous extent; K not a multiple of the 128-byte K tile, and for km_kn
    (no K-contiguous operand) not even of a 16-byte vector."""
    for (M, N, K) in [(144, 112, 208), (80, 336, 80)] + ([(96, 160, 77), (64, 64, 1)] if layout == "km_kn" else []):
        a_st, b_st, a_mk, b_kn = _operands(kind, layout, M, N, K, 1200 + K, pad_a=16, pad_b=32)
        _check(kind, _run(kind, layout, a_st, b_st, M, N, K), a_mk, b_kn)


def test_layouts_passthrough_int8_keeps_the_low_byte():
    M, N, K = 128, 96, 512
    a_st, b_st, a_mk, b_kn = _operands("i8", "km_kn", M, N, K, 5)
    _check("i8", _run("i8", "km_kn", a_st, b_st, M, N, K), a_mk, b_kn)


@pytest.mark.parametrize("layout", sorted(LAYOUTS))
def test_layouts_position_sensitive_operands(layout):
    """A = one-hot rows, B = distinct small integers: C must be an exact row selection of B, so a fragment
    that lands on the wrong row, column or k shows up as a wrong value, not as a tolerance question."""
    M, N, K = 320, 272, 192
    al, bl = LAYOUTS[layout]
    a_mk = np.zeros((M, K), np.float16)
    sel = (np.arange(M) * 7 + 3) % K
    a_mk[np.arange(M), sel] = 1
    b_kn = ((np.arange(K)[:, None] * 31 + np.arange(N)[None, :] * 17) % 2039).astype(np.float16)   # < 2048: exact
    a_st = np.ascontiguousarray(a_mk.T) if al is ck.ColumnMajor else a_mk
    b_st = b_kn if bl is ck.RowMajor else np.ascontiguousarray(b_kn.T)
    for instance in [capi.INSTANCE_AUTO] + TILES:
        out = _run("f16", layout, a_st, b_st, M, N, K, instance)
        np.testing.assert_array_equal(out, b_kn[sel, :])


@pytest.mark.parametrize("layout", sorted(LAYOUTS))
@pytest.mark.parametrize("kind", ["i8", "f16", "bf16"])
def test_layouts_large_problem_and_split_k(kind, layout, force_k_runs):
    M, N, K = 1024, 768, 2048
    a_st, b_st, a_mk, b_kn = _operands(kind, layout, M, N, K, 1300)
    c_op = ck.RequantReluRequant(0.002, 0.9, rounded=True) if kind == "i8" else None
    _check(kind, _run(kind, layout, a_st, b_st, M, N, K, c_op=c_op), a_mk, b_kn, c_op, big=True)
    force_k_runs(4)
    _check(kind, _run(kind, layout, a_st, b_st, M, N, K, c_op=c_op, workspace=True), a_mk, b_kn, c_op, big=True)


@pytest.mark.parametrize("layout", sorted(LAYOUTS))
def test_layouts_explicit_kbatch(layout):
    M, N, K = 192, 208, 1536
    a_st, b_st, a_mk, b_kn = _operands("i8", layout, M, N, K, 1400)
    c_op = ck.RequantReluRequant(0.01, 0.5, rounded=True)
    _check("i8", _run("i8", layout, a_st, b_st, M, N, K, c_op=c_op, k_batch=3), a_mk, b_kn, c_op)
    a_st, b_st, a_mk, b_kn = _operands("f16", layout, M, N, K, 1401)
    _check("f16", _run("f16", layout, a_st, b_st, M, N, K, k_batch=4), a_mk, b_kn)


@pytest.mark.parametrize("layout", sorted(LAYOUTS))
def test_layouts_refused_arguments(layout):
    M, N, K = 64, 64, 64
    a_st, b_st, _, _ = _operands("i8", layout, M, N, K, 7)
    n_tiles = 9
    for instance in (5, 6, n_tiles, n_tiles + 4):          # tiles of 32 / 16 rows, skinny instances
        _run("i8", layout, a_st, b_st, M, N, K, instance, expect_unsupported=True)
    al, bl = LAYOUTS[layout]
    # contiguous extent of the K-major operand not a whole 16-byte vector: refused by the vectorised tile instances,
    # taken by the element-wise instance and by the automatic choice; a stride below the extent by nobody
    lib = capi.lib()
    if al is ck.ColumnMajor:
        assert lib.ckx_gemm_f16_is_supported(60, 64, 64, 64, 64, 64, al.code, bl.code, ck.RowMajor.code, 0) == capi.UNSUPPORTED
        assert lib.ckx_gemm_f16_is_supported(60, 64, 64, 64, 64, 64, al.code, bl.code, ck.RowMajor.code, -1) == capi.OK
        assert lib.ckx_gemm_f16_is_supported(64, 64, 64, 60, 64, 64, al.code, bl.code, ck.RowMajor.code, -1) == capi.UNSUPPORTED
    if bl is ck.RowMajor:
        assert lib.ckx_gemm_i8_is_supported(64, 72, 64, 64, 80, 72, al.code, bl.code, ck.RowMajor.code, 0, 0) == capi.UNSUPPORTED
        assert lib.ckx_gemm_i8_is_supported(64, 72, 64, 64, 80, 72, al.code, bl.code, ck.RowMajor.code, 0, -1) == capi.OK
    # column-major C is in none of the reference's instance lists either
    assert lib.ckx_gemm_f16_is_supported(64, 64, 64, 64, 64, 64, al.code, bl.code, ck.ColumnMajor.code, -1) == capi.UNSUPPORTED


@pytest.mark.parametrize("layout", sorted(LAYOUTS))
def test_batched_gemm_layouts(layout):
    import torch
    import gpu_util
    G, M, N, K = 5, 144, 208, 320
    al, bl = LAYOUTS[layout]
    outs, refs = [], []
    a_all, b_all = [], []
    for g in range(G):
        a_st, b_st, a_mk, b_kn = _operands("f16", layout, M, N, K, 1500 + 2 * g)
        a_all.append(a_st), b_all.append(b_st)
        refs.append(lit.gemm_f16(a_mk, b_kn))
    da = torch.from_numpy(np.stack(a_all).view(np.int16)).cuda()
    db = torch.from_numpy(np.stack(b_all).view(np.int16)).cuda()
    dc = torch.full((G, M, N), 0x7E00, dtype=torch.int16, device="cuda")
    op = ck.DeviceBatchedGemmF16(capi.INSTANCE_AUTO, ALayout=al, BLayout=bl)
    arg = op.MakeArgumentPointer(da, db, dc, M, N, K, a_all[0].shape[1], b_all[0].shape[1], N, M * K, N * K, M * N, G)
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    out = dc.cpu().numpy().view(np.float16)
    for g in range(G):
        bad, max_err = lit.check_err_f16(out[g], refs[g], 1e-2, 1e-2)
        assert bad == 0, f"batch {g}: {bad} outside tolerance, max err {max_err}"


@pytest.mark.parametrize("layout", sorted(LAYOUTS))
def test_fp16_layouts_integer_operands_bit_exact_2048(layout):
    """Integers in [-5, 5]: fp32 accumulation is exact in any order (|sum| <= 25 * 2048 < 2^24), so the fp16 output of
    the transposing-read paths must equal the rounded exact product bit for bit."""
    M = N = K = 2048
    al, bl = LAYOUTS[layout]
    a_mk = uniform_int8((M, K), -5, 5, 71).astype(np.float32)
    b_kn = uniform_int8((K, N), -5, 5, 72).astype(np.float32)
    a_st = (a_mk.T if al is ck.ColumnMajor else a_mk).astype(np.float16)
    b_st = (b_kn if bl is ck.RowMajor else b_kn.T).astype(np.float16)
    out = _run("f16", layout, np.ascontiguousarray(a_st), np.ascontiguousarray(b_st), M, N, K)
    np.testing.assert_array_equal(out, (a_mk @ b_kn).astype(np.float16))
