"""GPU parity on seeded random problems: GEMM shapes, leading dimensions, layouts, epilogues and instances drawn at
random (ragged M / N, K tails, padded rows), and conv geometries with 1, 2 and 3 spatial dimensions -- every draw
through the C ABI against the CPU oracle's BLAS forms (bit-exact for int8, rtol = atol = 1e-2 for fp16).
The reference's own tests use fixed shapes (test/gemm/gemm_util.hpp, test/convnd_fwd/*.cpp); the draws here go
after what fixed shapes miss: tails in every dimension at once, odd strides, instance / layout combinations."""
import ctypes as C

import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from oracle import fast, lit

pytestmark = pytest.mark.gpu
LAYOUT_CODES = {"mk_nk": (ck.RowMajor, ck.ColumnMajor), "km_kn": (ck.ColumnMajor, ck.RowMajor),
                "km_nk": (ck.ColumnMajor, ck.ColumnMajor), "mk_kn": (ck.RowMajor, ck.RowMajor)}


def _draw_gemm(rng, kind):
    es = 1 if kind == "i8" else 2
    v = 16 // es                                   # elements of a 16-byte vector
    layout = rng.choice(sorted(LAYOUT_CODES))
    al, bl = LAYOUT_CODES[layout]
    M, N = int(rng.integers(1, 600)), int(rng.integers(1, 600))
    K = int(rng.integers(1, 96)) * v
    # the contiguous extent of a K-major operand is a whole number of vectors
    if al is ck.ColumnMajor:
        M = -(-M // v) * v
    if bl is ck.RowMajor:
        N = -(-N // v) * v
    pad_a, pad_b = int(rng.integers(0, 3)) * v, int(rng.integers(0, 3)) * v
    ldc = N + int(rng.integers(0, 3)) * v
    return layout, M, N, K, pad_a, pad_b, ldc


@pytest.mark.parametrize("seed", range(150))
@pytest.mark.parametrize("kind", ["i8", "f16"])
def test_random_gemm(kind, seed):
    import torch
    import gpu_util
    rng = np.random.default_rng(7000 + seed + (1000 if kind == "f16" else 0))
    layout, M, N, K, pad_a, pad_b, ldc = _draw_gemm(rng, kind)
    al, bl = LAYOUT_CODES[layout]
    gen = (lambda s: rng.integers(-8, 9, s).astype(np.int8)) if kind == "i8" else \
          (lambda s: rng.uniform(-1, 1, s).astype(np.float16))
    a_st = gen((K, M + pad_a) if al is ck.ColumnMajor else (M, K + pad_a))
    b_st = gen((K, N + pad_b) if bl is ck.RowMajor else (N, K + pad_b))
    a_mk = a_st[:, :M].T if al is ck.ColumnMajor else a_st[:, :K]
    b_kn = b_st[:, :N] if bl is ck.RowMajor else b_st[:, :K].T
    n_inst = capi.lib().ckx_num_instances(capi.OP_GEMM_I8)
    instance = int(rng.integers(-1, n_inst))
    c_op = None
    if kind == "i8":
        c_op = [None, ck.RequantReluRequant(0.03, 0.6, rounded=True), ck.RequantReluRequant(0.05, 1.0)][int(rng.integers(0, 3))]
    raw = (lambda x: x) if kind == "i8" else (lambda x: x.view(np.int16))
    da, db = (torch.from_numpy(raw(np.ascontiguousarray(x))).cuda() for x in (a_st, b_st))
    dc = torch.full((M, ldc), 77 if kind == "i8" else 0x7E00, dtype=torch.int8 if kind == "i8" else torch.int16, device="cuda")
    op = (ck.DeviceGemmInt8 if kind == "i8" else ck.DeviceGemmF16)(instance, ALayout=al, BLayout=bl)
    arg = op.MakeArgumentPointer(da, db, dc, M, N, K, a_st.shape[1], b_st.shape[1], ldc, None, None, c_op)
    desc = f"{kind} {layout} M{M} N{N} K{K} lda{a_st.shape[1]} ldb{b_st.shape[1]} ldc{ldc} inst{instance} op{c_op}"
    if not op.IsSupportedArgument(arg):
        # only an instance that does not cover the shape or layout may refuse; the automatic choice never does
        assert instance != capi.INSTANCE_AUTO, desc + ": " + capi.last_error().decode()
        return
    if rng.integers(0, 2):
        ws = torch.full((max(op.GetWorkSpaceSize(arg), 16),), 0x7F, dtype=torch.uint8, device="cuda")
        op.SetWorkSpacePointer(arg, ws)
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    out = dc.cpu().numpy()
    if kind == "i8":
        assert np.all(out[:, N:] == 77), desc + ": wrote outside the C rows"
        epi = (lit.EPI_PASSTHROUGH, 1.0, 1.0) if c_op is None else \
              (lit.EPI_REQUANT_RND if c_op.epilogue == capi.EPI_REQUANT_RND else lit.EPI_REQUANT_CK, c_op.scale_gemm, c_op.scale_relu)
        np.testing.assert_array_equal(out[:, :N], fast.gemm_i8(a_mk, b_kn, *epi), err_msg=desc)
    else:
        assert np.all(out[:, N:] == 0x7E00), desc + ": wrote outside the C rows"
        bad, max_err = lit.check_err_f16(np.ascontiguousarray(out[:, :N]).view(np.float16), fast.gemm_f16(a_mk, b_kn), 1e-2, 1e-2)
        assert bad == 0, f"{desc}: {bad} outside tolerance, max err {max_err}"


@pytest.mark.parametrize("seed", range(150))
@pytest.mark.parametrize("kind", ["i8", "f16"])
def test_random_conv(kind, seed):
    import gpu_util
    rng = np.random.default_rng(9000 + seed + (1000 if kind == "f16" else 0))
    nd = int(rng.integers(1, 4))
    es = 1 if kind == "i8" else 2
    Cc = int(rng.integers(1, 5)) * (16 // es)
    K = int(rng.integers(1, 100))
    N = int(rng.integers(1, 4))
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
    n_tiles = capi.lib().ckx_num_instances(capi.OP_GEMM_SPLITK)      # the tile instances: valid for every conv
    instance = int(rng.integers(-1, n_tiles))
    desc = f"{kind} nd{nd} N{N} C{Cc} K{K} in{in_len} f{filt} s{st} d{dil} p{pad}/{rpad} inst{instance}"
    rq = ck.RequantReluRequant(0.05, 0.7, rounded=True) if kind == "i8" and rng.integers(0, 2) else None
    out = gpu_util.convnd_fwd(inp, wei, st, dil, pad, out_op=rq, instance=instance, right_pads=rpad,
                              workspace=bool(rng.integers(0, 2)))
    if kind == "i8":
        epi = dict(epi=lit.EPI_REQUANT_RND, scale_gemm=0.05, scale_relu=0.7) if rq else {}
        np.testing.assert_array_equal(out, fast.convnd_fwd(inp, wei, st, dil, pad, rpad, **epi), err_msg=desc)
    else:
        bad, max_err = lit.check_err_f16(out, fast.convnd_fwd(inp, wei, st, dil, pad, rpad), 1e-2, 1e-2)
        assert bad == 0, f"{desc}: {bad} outside tolerance, max err {max_err}"


@pytest.mark.parametrize("seed", range(80))
def test_random_gemm_gemm(seed):
    """Fused GEMM-GEMM and GEMM-softmax-GEMM: random batch / row / column counts (ragged slabs and steps, one to
    many 128-column steps), K and O at every multiple of 8 up to 128, padded strides, scale sign, mask, instance."""
    import torch
    import gpu_util
    rng = np.random.default_rng(11000 + seed)
    G, M, N = int(rng.integers(1, 5)), int(rng.integers(1, 300)), int(rng.integers(1, 700))
    K, O = 8 * int(rng.integers(1, 17)), 8 * int(rng.integers(1, 17))
    softmax = bool(rng.integers(0, 2))
    mask = softmax and bool(rng.integers(0, 2))
    scale = float(rng.choice([1.0, -0.7, 0.25])) / np.sqrt(K) if softmax else 1.0
    instance = int(rng.integers(-1, capi.lib().ckx_num_instances(capi.OP_BATCHED_GEMM_GEMM)))
    pad = [8 * int(rng.integers(0, 3)) for _ in range(4)]
    lim = 1.0 if softmax else 0.5
    a, b0, b1 = (rng.uniform(-lim, lim, s).astype(np.float16) for s in ((G, M, K), (G, N, K), (G, N, O)))

    def padded(x, p):
        out = np.zeros(x.shape[:2] + (x.shape[2] + p,), np.float16)
        out[..., :x.shape[2]] = x
        return out

    ha, hb0, hb1 = padded(a, pad[0]), padded(b0, pad[1]), padded(b1, pad[2])
    da, db0, db1 = (torch.from_numpy(x.view(np.int16)).cuda() for x in (ha, hb0, hb1))
    dc = torch.full((G, M, O + pad[3]), 0x7E00, dtype=torch.int16, device="cuda")
    dims = (M, N, K, O, G, K + pad[0], K + pad[1], O + pad[2], O + pad[3], M * (K + pad[0]), N * (K + pad[1]),
            N * (O + pad[2]), M * (O + pad[3]))
    if softmax:
        op = ck.DeviceBatchedGemmSoftmaxGemmF16(instance, MaskOutUpperTriangle=mask)
        arg = op.MakeArgumentPointer(da, db0, db1, dc, *dims, None, None, ck.Scale(scale))
        ref = lit.batched_gemm_softmax_gemm_f16(a, b0.transpose(0, 2, 1), b1, scale, mask)
    else:
        op = ck.DeviceBatchedGemmGemmF16(instance)
        arg = op.MakeArgumentPointer(da, db0, db1, dc, *dims)
        ref = lit.batched_gemm_gemm_f16(a, b0.transpose(0, 2, 1), b1)
    desc = f"G{G} M{M} N{N} K{K} O{O} softmax{softmax} mask{mask} scale{scale:.3f} inst{instance} pad{pad}"
    assert op.IsSupportedArgument(arg), desc + ": " + capi.last_error().decode()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    out = dc.cpu().numpy().view(np.float16)
    assert np.all(out[..., O:].view(np.uint16) == 0x7E00), desc + ": wrote outside the C rows"
    bad, max_err = lit.check_err_f16(np.ascontiguousarray(out[..., :O]), ref, 1e-2, 1e-2)
    assert bad == 0, f"{desc}: {bad} outside tolerance, max err {max_err}"
