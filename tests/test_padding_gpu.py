"""GPU parity of the element-granular instance, through the C ABI: what the reference covers with its padded GEMM
instances (GemmSpecialization::KPadding / MNKPadding, gemm_specialization.hpp:10-20) and its odd-channel conv
instances (ConvolutionForwardSpecialization::OddC; device test case C = 3, test/convnd_fwd/conv2d_fwd.cpp:111):
K, leading dimensions, channel counts and base addresses that are not whole 16-byte vectors. The automatic choice
must take every such problem; int8 is bit-exact against the oracle, fp16 / bf16 within rtol = atol = 1e-2."""
import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8
from oracle import fast, lit

pytestmark = pytest.mark.gpu

LAYOUTS = {"mk_nk": (ck.RowMajor, ck.ColumnMajor), "km_kn": (ck.ColumnMajor, ck.RowMajor),
           "km_nk": (ck.ColumnMajor, ck.ColumnMajor), "mk_kn": (ck.RowMajor, ck.RowMajor)}
NP_T = {"i8": np.int8, "f16": np.float16, "bf16": np.uint16}


def _generic():
    L = capi.lib()
    n = L.ckx_num_instances(capi.OP_GEMM_I8)
    assert b"Generic" in L.ckx_instance_name(capi.OP_GEMM_I8, n - 1)
    return n - 1


def _f16_close(out, ref):
    bad, max_err = lit.check_err_f16(out, ref, 1e-2, 1e-2)
    assert bad == 0, f"{bad} outside tolerance, max err {max_err}"


def _gemm(kind, layout, a_st, b_st, M, N, K, ldc=None, c_op=None, instance=capi.INSTANCE_AUTO, off_a=0, off_b=0):
    """a_st / b_st: operands as stored (2-D); off_a / off_b: elements by which the device copy is shifted from its
    (256-byte aligned) allocation, so that the base address is not a vector boundary either."""
    import torch
    import gpu_util
    es = 1 if kind == "i8" else 2
    tdt = torch.int8 if kind == "i8" else torch.int16
    raw = (lambda x: np.ascontiguousarray(x)) if kind == "i8" else (lambda x: np.ascontiguousarray(x).view(np.int16))

    def shifted(x, off):
        buf = torch.zeros(x.size + off, dtype=tdt, device="cuda")
        buf[off:] = torch.from_numpy(raw(x)).cuda().reshape(-1)
        return buf, buf.data_ptr() + off * es

    ba, pa = shifted(a_st, off_a)
    bb, pb = shifted(b_st, off_b)
    ldc = ldc or N
    dc = torch.full((M, ldc), 77 if kind == "i8" else 0x7E00, dtype=tdt, device="cuda")
    al, bl = LAYOUTS[layout]
    cls = {"i8": ck.DeviceGemmInt8, "f16": ck.DeviceGemmF16, "bf16": ck.DeviceGemmBF16}[kind]
    op = cls(instance, ALayout=al, BLayout=bl)
    arg = op.MakeArgumentPointer(pa, pb, dc, M, N, K, a_st.shape[1], b_st.shape[1], ldc, None, None, c_op)
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    out = dc.cpu().numpy()
    assert np.all(out[:, N:] == (77 if kind == "i8" else 0x7E00)), "wrote outside the C rows"
    out = np.ascontiguousarray(out[:, :N])
    return out if kind == "i8" else out.view(np.float16 if kind == "f16" else np.uint16)


@pytest.mark.parametrize("shape", [(64, 64, 100), (130, 70, 100), (1, 1, 1), (300, 17, 1003), (16, 250, 4099)])
@pytest.mark.parametrize("explicit", [False, True])
def test_int8_gemm_k_not_a_vector_bit_exact(shape, explicit):
    """K = 100 and friends against the literal ReferenceGemm restatement, all three int8 epilogues."""
    M, N, K = shape
    a, b_nk = uniform_int8((M, K), -8, 8, 2000 + K), uniform_int8((N, K), -8, 8, 2001 + M)
    inst = _generic() if explicit else capi.INSTANCE_AUTO
    for c_op, epi in ((None, (lit.EPI_PASSTHROUGH, 1.0, 1.0)),
                      (ck.RequantReluRequant(0.02, 0.4, rounded=True), (lit.EPI_REQUANT_RND, 0.02, 0.4)),
                      (ck.RequantReluRequant(0.03, 1.0), (lit.EPI_REQUANT_CK, 0.03, 1.0))):
        out = _gemm("i8", "mk_nk", a, b_nk, M, N, K, c_op=c_op, instance=inst)
        np.testing.assert_array_equal(out, lit.gemm_i8(a, b_nk.T, *epi))


@pytest.mark.parametrize("shape", [(96, 80, 1001), (64, 64, 60), (7, 5, 3), (257, 129, 33)])
def test_fp16_gemm_k_not_a_vector(shape):
    M, N, K = shape
    a, b_nk = uniform_f16((M, K), -1, 1, 2010 + K), uniform_f16((N, K), -1, 1, 2011 + M)
    _f16_close(_gemm("f16", "mk_nk", a, b_nk, M, N, K), lit.gemm_f16(a, b_nk.T))
    # small integers: every partial sum is exact in fp32, the result must be the rounded exact product
    ai, bi = uniform_int8((M, K), -5, 5, 2012).astype(np.float16), uniform_int8((N, K), -5, 5, 2013).astype(np.float16)
    exact = ai.astype(np.float32) @ bi.astype(np.float32).T
    np.testing.assert_array_equal(_gemm("f16", "mk_nk", ai, bi, M, N, K), exact.astype(np.float16))


@pytest.mark.parametrize("seed", range(40))
@pytest.mark.parametrize("kind", ["i8", "f16", "bf16"])
def test_random_ragged_gemm(kind, seed):
    """Every extent, leading dimension and base address drawn element-granular, all four layouts."""
    rng = np.random.default_rng(21000 + seed + {"i8": 0, "f16": 100, "bf16": 200}[kind])
    layout = str(rng.choice(sorted(LAYOUTS)))
    al, bl = LAYOUTS[layout]
    M, N, K = (int(rng.integers(1, 200)) for _ in range(3))
    pad_a, pad_b, pad_c = (int(rng.integers(0, 6)) for _ in range(3))
    off_a, off_b = int(rng.integers(0, 4)), int(rng.integers(0, 4))
    if kind == "i8":
        gen = lambda s: rng.integers(-8, 9, s).astype(np.int8)
    elif kind == "f16":
        gen = lambda s: rng.uniform(-1, 1, s).astype(np.float16)
    else:
        gen = lambda s: fast.f32_to_bf16(rng.uniform(-1, 1, s).astype(np.float32))
    a_st = gen((K, M + pad_a) if al is ck.ColumnMajor else (M, K + pad_a))
    b_st = gen((K, N + pad_b) if bl is ck.RowMajor else (N, K + pad_b))
    a_mk = a_st[:, :M].T if al is ck.ColumnMajor else a_st[:, :K]
    b_kn = b_st[:, :N] if bl is ck.RowMajor else b_st[:, :K].T
    c_op = ck.RequantReluRequant(0.03, 0.6, rounded=True) if kind == "i8" and rng.integers(0, 2) else None
    out = _gemm(kind, layout, a_st, b_st, M, N, K, ldc=N + pad_c, c_op=c_op, off_a=off_a, off_b=off_b)
    desc = f"{kind} {layout} M{M} N{N} K{K} pads {pad_a},{pad_b},{pad_c} offsets {off_a},{off_b}"
    if kind == "i8":
        epi = (lit.EPI_REQUANT_RND, 0.03, 0.6) if c_op else (lit.EPI_PASSTHROUGH, 1.0, 1.0)
        np.testing.assert_array_equal(out, fast.gemm_i8(a_mk, b_kn, *epi), err_msg=desc)
    elif kind == "f16":
        _f16_close(out, fast.gemm_f16(a_mk, b_kn))
    else:
        o, r = fast.bf16_to_f32(out), fast.bf16_to_f32(fast.gemm_bf16(a_mk, b_kn))
        assert np.all(np.abs(o - r) <= 1e-2 + 1e-2 * np.abs(r)), desc


def test_batched_gemm_ragged_k_and_batch_strides():
    import torch
    import gpu_util
    G, M, N, K = 5, 70, 45, 100
    bsa, bsb, bsc = M * K + 3, N * K + 1, M * N + 7
    a = uniform_int8((G, bsa), -8, 8, 2100)
    b = uniform_int8((G, bsb), -8, 8, 2101)
    da, db = gpu_util.dev(a), gpu_util.dev(b)
    dc = torch.full((G, bsc), 77, dtype=torch.int8, device="cuda")
    op = ck.DeviceBatchedGemmInt8()
    c_op = ck.RequantReluRequant(0.02, 0.4, rounded=True)
    arg = op.MakeArgumentPointer(da, db, dc, M, N, K, K, K, N, bsa, bsb, bsc, G, None, None, c_op)
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    out = dc.cpu().numpy()
    for g in range(G):
        a_g, b_g = a[g, :M * K].reshape(M, K), b[g, :N * K].reshape(N, K)
        np.testing.assert_array_equal(out[g, :M * N].reshape(M, N), lit.gemm_i8(a_g, b_g.T, lit.EPI_REQUANT_RND, 0.02, 0.4))
        assert np.all(out[g, M * N:] == 77)


@pytest.mark.parametrize("layout", ["mk_nk", "km_kn"])
def test_gemm_with_d_operands_on_ragged_shapes(layout):
    """AddRelu on the fp16-rounded C (example 03) and AddReluAdd, K = 100, N = 50, also on K-major operands."""
    import torch
    import gpu_util
    M, N, K = 90, 50, 100
    al, bl = LAYOUTS[layout]
    a_mk, b_kn = uniform_f16((M, K), -1, 1, 2200), uniform_f16((K, N), -1, 1, 2201)
    a_st = np.ascontiguousarray(a_mk.T) if al is ck.ColumnMajor else a_mk
    b_st = b_kn if bl is ck.RowMajor else np.ascontiguousarray(b_kn.T)
    bias, resi = uniform_f16((N,), -1, 1, 2202), uniform_f16((M, N), -1, 1, 2203)
    acc = a_mk.astype(np.float32) @ b_kn.astype(np.float32)
    da, db, dbias, dresi = (gpu_util.dev(x) for x in (a_st, b_st, bias, resi))
    for functor, ds, strides, want in (
            (ck.AddRelu(), [dbias], [0],
             np.maximum((acc.astype(np.float16).astype(np.float32) + bias.astype(np.float32)).astype(np.float16), 0)),
            (ck.AddReluAdd(), [dbias, dresi], [0, N],
             (np.maximum(acc + bias.astype(np.float32), 0) + resi.astype(np.float32)).astype(np.float16))):
        de = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        op = ck.DeviceGemmMultipleDF16(capi.INSTANCE_AUTO, ALayout=al, BLayout=bl)
        arg = op.MakeArgumentPointer(da, db, ds, de, M, N, K, a_st.shape[1], b_st.shape[1], strides, N, None, None, functor)
        assert op.IsSupportedArgument(arg), capi.last_error()
        op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
        torch.cuda.synchronize()
        _f16_close(de.cpu().numpy(), want)


@pytest.mark.parametrize("dtype", ["i8", "f16"])
def test_conv2d_odd_c_reference_device_test_case(dtype):
    """The reference's own odd-C device test case (test/convnd_fwd/conv2d_fwd.cpp:111): N 4, K 256, C 3, 3 x 3
    filter on 28 x 28, stride 1, no padding -- plus the same layer padded, strided and dilated."""
    import gpu_util
    for (s, d, p) in (((1, 1), (1, 1), (0, 0)), ((2, 1), (1, 2), (1, 2))):
        if dtype == "i8":
            inp, wei = uniform_int8((4, 28, 28, 3), -5, 5, 2300), uniform_int8((256, 3, 3, 3), -5, 5, 2301)
            out = gpu_util.conv2d_fwd(inp, wei, s, d, p)
            np.testing.assert_array_equal(out, fast.conv2d_fwd_i8(inp, wei, s, d, p))
            np.testing.assert_array_equal(out[:1], lit.conv2d_fwd(inp[:1], wei, s, d, p))
            rq = ck.RequantReluRequant(0.05, 0.7, rounded=True)
            out = gpu_util.conv2d_fwd(inp, wei, s, d, p, out_op=rq)
            np.testing.assert_array_equal(out, fast.conv2d_fwd_i8(inp, wei, s, d, p, epi=lit.EPI_REQUANT_RND,
                                                                  scale_gemm=0.05, scale_relu=0.7))
        else:
            inp, wei = uniform_f16((4, 28, 28, 3), -1, 1, 2302), uniform_f16((256, 3, 3, 3), -1, 1, 2303)
            out = gpu_util.conv2d_fwd(inp, wei, s, d, p)
            _f16_close(out, fast.conv2d_fwd_f16(inp, wei, s, d, p))
            _f16_close(out[:1], lit.conv2d_fwd(inp[:1], wei, s, d, p))


@pytest.mark.parametrize("seed", range(40))
@pytest.mark.parametrize("kind", ["i8", "f16"])
def test_random_conv_any_channel_count(kind, seed):
    """1, 2 and 3 spatial dimensions with channel counts that are not whole vectors."""
    import gpu_util
    rng = np.random.default_rng(23000 + seed + (1000 if kind == "f16" else 0))
    nd = int(rng.integers(1, 4))
    Cc, K, N = int(rng.integers(1, 40)), int(rng.integers(1, 100)), int(rng.integers(1, 4))
    filt = [int(rng.integers(1, 4)) for _ in range(nd)]
    dil = [int(rng.integers(1, 3)) for _ in range(nd)]
    st = [int(rng.integers(1, 3)) for _ in range(nd)]
    pad = [int(rng.integers(0, 3)) for _ in range(nd)]
    rpad = [int(rng.integers(0, 3)) for _ in range(nd)]
    hi = {1: 60, 2: 14, 3: 7}[nd]
    in_len = [max(int(rng.integers(1, hi)), (filt[i] - 1) * dil[i] + 1 - pad[i] - rpad[i]) for i in range(nd)]
    gen = (lambda s: rng.integers(-5, 6, s).astype(np.int8)) if kind == "i8" else \
          (lambda s: rng.uniform(-1, 1, s).astype(np.float16))
    inp, wei = gen((N, *in_len, Cc)), gen((K, *filt, Cc))
    desc = f"{kind} nd{nd} N{N} C{Cc} K{K} in{in_len} f{filt} s{st} d{dil} p{pad}/{rpad}"
    rq = ck.RequantReluRequant(0.05, 0.7, rounded=True) if kind == "i8" and rng.integers(0, 2) else None
    out = gpu_util.convnd_fwd(inp, wei, st, dil, pad, out_op=rq, right_pads=rpad)
    if kind == "i8":
        epi = dict(epi=lit.EPI_REQUANT_RND, scale_gemm=0.05, scale_relu=0.7) if rq else {}
        np.testing.assert_array_equal(out, fast.convnd_fwd(inp, wei, st, dil, pad, rpad, **epi), err_msg=desc)
    else:
        bad, max_err = lit.check_err_f16(out, fast.convnd_fwd(inp, wei, st, dil, pad, rpad), 1e-2, 1e-2)
        assert bad == 0, f"{desc}: {bad} outside tolerance, max err {max_err}"


def test_conv2d_bias_relu_add_with_odd_c():
    import torch
    import gpu_util
    N, C, K, Hi, Wi = 2, 3, 20, 9, 11
    s, d, p = (1, 1), (1, 1), (1, 1)
    inp, wei = uniform_f16((N, Hi, Wi, C), -1, 1, 2400), uniform_f16((K, 3, 3, C), -1, 1, 2401)
    bias, resi = uniform_f16((K,), -1, 1, 2402), uniform_f16((N, Hi, Wi, K), -1, 1, 2403)
    di, dw, db, dr = (gpu_util.dev(x) for x in (inp, wei, bias, resi))
    do = torch.full((N, Hi, Wi, K), float("nan"), dtype=torch.float16, device="cuda")
    op = ck.DeviceConv2dFwdBiasActivationF16()
    arg = op.MakeArgumentPointer(di, dw, do, db, dr, N, K, C, [Hi, Wi], [3, 3], [Hi, Wi], list(s), list(d), list(p),
                                 list(p), None, None, ck.AddReluAdd())
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    _f16_close(do.cpu().numpy(), lit.conv2d_fwd_bias_relu_f16(inp, wei, bias, resi, s, d, p))
