"""GPU tests of the C++ host layer: the ckProfiler-style driver and the example that mirrors the
reference's example 14 run as child processes; the tensors they write are checked against the
CPU oracle on inputs regenerated here from the same seeds (the generators are counter based)."""
import os
import subprocess

import numpy as np
import pytest

from composable_kernel_amd.host_tensor import uniform_f16, uniform_int8
from oracle import fast, lit

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "composable_kernel_amd", "bin")
SEED = 0xC0FFEE


def _run(exe, args, dump_var, tmp_path):
    path = os.path.join(BIN, exe)
    if not os.path.exists(path):
        pytest.fail(f"{path} is not built (python -m composable_kernel_amd.build)")
    dump = str(tmp_path / "out.bin")
    env = dict(os.environ, **{dump_var: dump})
    r = subprocess.run([path] + [str(a) for a in args], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True, timeout=300)
    assert r.returncode == 0, r.stdout
    return r.stdout, dump


def test_profiler_int8_requant_gemm_all_instances_agree_and_match_oracle(tmp_path):
    M, N, K = 1024, 1024, 1024
    out, dump = _run("ckx_profiler", ["gemm", 3, 1, 1, 1, 0, 1, M, N, K, -1, -1, -1, 2, 0.5, 0.03], "CKX_PROFILER_DUMP",
                     tmp_path)
    assert "Best Perf:" in out and "Error" not in out
    assert out.count("Perf:") >= 8
    c = np.fromfile(dump, np.int8).reshape(M, N)
    a = uniform_int8((M, K), -5, 5, SEED)
    b_nk = uniform_int8((N, K), -5, 5, SEED + 1)
    np.testing.assert_array_equal(c, lit.gemm_i8(a, b_nk.T, lit.EPI_REQUANT_RND, 0.5, 0.03))


def test_profiler_fp16_gemm(tmp_path):
    M, N, K = 512, 768, 1024
    out, dump = _run("ckx_profiler", ["gemm", 1, 1, 1, 2, 0, 1, M, N, K, -1, -1, -1], "CKX_PROFILER_DUMP", tmp_path)
    assert "Best Perf:" in out and "Error" not in out
    c = np.fromfile(dump, np.float16).reshape(M, N)
    a = uniform_f16((M, K), -1, 1, SEED)
    b_nk = uniform_f16((N, K), -1, 1, SEED + 1)
    bad, max_err = lit.check_err_f16(c, lit.gemm_f16(a, b_nk.T), 1e-2, 1e-2)
    assert bad == 0, max_err


def test_profiler_conv2d_fwd_int8(tmp_path):
    # N K C Y X Hi Wi Sy Sx Dy Dx LPy LPx RPy RPx (the reference's argument order)
    geo = [4, 64, 32, 3, 3, 14, 14, 2, 2, 1, 1, 1, 1, 1, 1]
    out, dump = _run("ckx_profiler", ["conv2d_fwd", 3, 1, 1, 0, 1] + geo, "CKX_PROFILER_DUMP", tmp_path)
    assert "Best Perf:" in out and "Error" not in out
    N, K, C, Y, X, Hi, Wi = geo[:7]
    inp = uniform_int8((N, Hi, Wi, C), -5, 5, SEED + 2)
    wei = uniform_int8((K, Y, X, C), -5, 5, SEED + 3)
    want = lit.conv2d_fwd(inp, wei, (2, 2), (1, 1), (1, 1))
    c = np.fromfile(dump, np.int8).reshape(want.shape)
    np.testing.assert_array_equal(c, want)


@pytest.mark.parametrize("ndim", [1, 3])
def test_profiler_convnd_fwd_int8(tmp_path, ndim):
    """profile_convnd_fwd's argument order (profiler/src/profile_convnd_fwd.cpp:81-115): data type, layout, verify,
    init, log, repeats, NDim, then N K C <filter> <input> <strides> <dilations> <left pads> <right pads>."""
    if ndim == 1:
        filt, inp_len, st, dl, pd = [3], [40], [2], [2], [2]
    else:
        filt, inp_len, st, dl, pd = [3, 3, 3], [7, 9, 8], [2, 1, 2], [1, 2, 1], [1, 2, 1]
    N, K, C = 3, 64, 32
    out, dump = _run("ckx_profiler", ["convnd_fwd", 3, 1, 1, 1, 0, 3, ndim, N, K, C] + filt + inp_len + st + dl + pd + pd,
                     "CKX_PROFILER_DUMP", tmp_path)
    assert "Best Perf:" in out and "Error" not in out
    inp = uniform_int8((N, *inp_len, C), -5, 5, SEED + 2)
    wei = uniform_int8((K, *filt, C), -5, 5, SEED + 3)
    want = lit.convnd_fwd(inp, wei, st, dl, pd)
    np.testing.assert_array_equal(np.fromfile(dump, np.int8).reshape(want.shape), want)


def test_profiler_batched_gemm_gemm(tmp_path):
    M, N, K, O, G = 256, 384, 64, 64, 3
    out, dump = _run("ckx_profiler", ["batched_gemm_gemm", 1, 1, 0, 1, M, N, K, O, G], "CKX_PROFILER_DUMP", tmp_path)
    assert "Best Perf:" in out
    a = uniform_f16((G, M, K), -0.5, 0.5, SEED + 4)
    b0 = uniform_f16((G, N, K), -0.5, 0.5, SEED + 5)
    b1 = uniform_f16((G, N, O), -0.5, 0.5, SEED + 6)
    c = np.fromfile(dump, np.float16).reshape(G, M, O)
    bad, max_err = lit.check_err_f16(c, lit.batched_gemm_gemm_f16(a, b0.transpose(0, 2, 1), b1), 1e-2, 1e-2)
    assert bad == 0, max_err


def test_profiler_reports_unsupported_problems(tmp_path):
    """K = 100 is not a whole 16-byte vector: every vectorised instance says it does not support the problem (as the
    reference's profiler prints, profile_gemm_impl.hpp:205-208), the element-wise instance runs it; a leading
    dimension below K is supported by no instance and the profiler fails."""
    M, N, K = 64, 64, 100
    out, dump = _run("ckx_profiler", ["gemm", 3, 1, 1, 1, 0, 0, M, N, K, -1, -1, -1], "CKX_PROFILER_DUMP", tmp_path)
    assert out.count("does not support this problem") == 18      # the tile and skinny instances; the last one runs
    c = np.fromfile(dump, np.int8).reshape(M, N)
    a = uniform_int8((M, K), -5, 5, SEED)
    b_nk = uniform_int8((N, K), -5, 5, SEED + 1)
    np.testing.assert_array_equal(c, lit.gemm_i8(a, b_nk.T))
    path = os.path.join(BIN, "ckx_profiler")
    r = subprocess.run([path, "gemm", "3", "1", "0", "1", "0", "0", "64", "64", "100", "50", "-1", "-1"],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert r.returncode == 1
    assert "does not support this problem" in r.stdout and "no instance supports this problem" in r.stdout


def test_example_gemm_requant_relu_requant_int8(tmp_path):
    """Same call sequence and defaults as the reference's example 14 (scales 0.03 / 1, literal
    functor), on a smaller problem."""
    M, N, K = 768, 512, 1024
    out, dump = _run("example_gemm_requant_relu_requant_int8", [1, 1, 1, M, N, K, K, K, N], "CKX_EXAMPLE_DUMP", tmp_path)
    assert "Perf:" in out
    c = np.fromfile(dump, np.int8).reshape(M, N)
    a = uniform_int8((M, K), -5, 5, SEED)
    b_nk = uniform_int8((N, K), -5, 5, SEED + 1)
    want = lit.gemm_i8(a, b_nk.T, lit.EPI_REQUANT_CK, 0.03, 1.0)
    np.testing.assert_array_equal(c, want)
    assert f"sum(C) = {int(want.astype(np.int64).sum())}" in out


@pytest.mark.parametrize("with_resi", [False, True])
def test_profiler_conv_fwd_bias_relu_and_add(tmp_path, with_resi):
    """profile_conv_fwd_bias_relu[_add] of the reference's profiler (the ResNet-50 script's operations)."""
    geo = [2, 64, 32, 3, 3, 14, 14, 1, 1, 1, 1, 1, 1, 1, 1]
    op = "conv_fwd_bias_relu_add" if with_resi else "conv_fwd_bias_relu"
    out, dump = _run("ckx_profiler", [op, 1, 1, 2, 0, 1] + geo, "CKX_PROFILER_DUMP", tmp_path)
    assert "Best Perf:" in out and "Error" not in out and "AddRelu" in out
    N, K, C, Y, X, Hi, Wi = geo[:7]
    inp = uniform_f16((N, Hi, Wi, C), -1, 1, SEED + 2)
    wei = uniform_f16((K, Y, X, C), -1, 1, SEED + 3)
    bias = uniform_f16((K,), -1, 1, SEED + 7)
    resi = uniform_f16((N, 14, 14, K), -1, 1, SEED + 8) if with_resi else None
    want = lit.conv2d_fwd_bias_relu_f16(inp, wei, bias, resi, (1, 1), (1, 1), (1, 1))
    c = np.fromfile(dump, np.float16).reshape(want.shape)
    bad, max_err = lit.check_err_f16(c, want, 1e-2, 1e-2)
    assert bad == 0, max_err


def test_profiler_gemm_bias_relu(tmp_path):
    M, N, K = 384, 256, 512
    out, dump = _run("ckx_profiler", ["gemm_bias_relu", 1, 2, 0, 1, M, N, K], "CKX_PROFILER_DUMP", tmp_path)
    assert "Best Perf:" in out and "Error" not in out
    a = uniform_f16((M, K), -1, 1, SEED)
    b_nk = uniform_f16((N, K), -1, 1, SEED + 1)
    d = uniform_f16((N,), -1, 1, SEED + 9)
    c = np.fromfile(dump, np.float16).reshape(M, N)
    bad, max_err = lit.check_err_f16(c, lit.gemm_f16_add_relu(a, b_nk.T, d[None, :]), 1e-2, 1e-2)
    assert bad == 0, max_err


@pytest.mark.parametrize("layout", [1, 2])
def test_profiler_gemm_bilinear(tmp_path, layout):
    """profile_gemm_bilinear's argument list (alpha, beta = arg15, 16) over every instance of the C++
    DeviceGemmMultipleD<..., Tuple<half_t>, half_t, ..., Bilinear>; layout 2 stores A as [K, M] and B as [K, N]."""
    M, N, K = 320, 256, 512
    out, dump = _run("ckx_profiler", ["gemm_bilinear", 1, layout, 1, 2, 0, 1, M, N, K, -1, -1, -1, -1, 0.5, -1.25],
                     "CKX_PROFILER_DUMP", tmp_path)
    assert "Best Perf:" in out and "Error" not in out and "Bilinear" in out
    e = np.fromfile(dump, np.float16).reshape(M, N)
    a_st = uniform_f16((M, K) if layout == 1 else (K, M), -1, 1, SEED)
    b_st = uniform_f16((N, K) if layout == 1 else (K, N), -1, 1, SEED + 1)
    d = uniform_f16((M, N), -1, 1, SEED + 9)
    a_mk, b_kn = (a_st, b_st.T) if layout == 1 else (a_st.T, b_st)
    bad, max_err = lit.check_err_f16(e, fast.gemm_f16_bilinear(a_mk, b_kn, d, 0.5, -1.25), 1e-2, 1e-2)
    assert bad == 0, max_err


def test_profiler_gemm_add_add_fastgelu(tmp_path):
    """profile_gemm_add_add_fastgelu's argument list with example 04's strides: D0 a bias row (StrideD0 = 0), D1 dense."""
    M, N, K = 320, 256, 512
    out, dump = _run("ckx_profiler", ["gemm_add_add_fastgelu", 1, 1, 1, 2, 0, 1, M, N, K, -1, -1, 0, -1, -1],
                     "CKX_PROFILER_DUMP", tmp_path)
    assert "Best Perf:" in out and "Error" not in out and "AddAddFastGelu" in out
    e = np.fromfile(dump, np.float16).reshape(M, N)
    a = uniform_f16((M, K), -1, 1, SEED)
    b_nk = uniform_f16((N, K), -1, 1, SEED + 1)
    d0 = uniform_f16((N,), -1, 1, SEED + 9)
    d1 = uniform_f16((M, N), -1, 1, SEED + 10)
    bad, max_err = lit.check_err_f16(e, fast.gemm_f16_add_add_fastgelu(a, b_nk.T, d0[None, :], d1), 1e-2, 1e-2)
    assert bad == 0, max_err


@pytest.mark.parametrize("act", [0, 1])
def test_profiler_gemm_perchannel_quant(tmp_path, act):
    """C++ DeviceGemmMultipleD<int8, ..., Tuple<float>, int8, Activation_Mul2_Clamp<Act>> over every instance: all
    agree with the first, the best one matches the oracle bit for bit (init 1: int8 in [-5, 5]; the profiler's scale
    of column n is ((37 n) mod 61 - 20) / 256)."""
    M, N, K = 200, 320, 512
    out, dump = _run("ckx_profiler", ["gemm_perchannel_quant", 1, 1, 0, 1, M, N, K, -1, -1, -1, act], "CKX_PROFILER_DUMP",
                     tmp_path)
    assert "Best Perf:" in out and "Error" not in out and "Mul2_Clamp" in out
    e = np.fromfile(dump, np.int8).reshape(M, N)
    a = uniform_int8((M, K), -5, 5, SEED)
    b_nk = uniform_int8((N, K), -5, 5, SEED + 1)
    scale = (((np.arange(N) * 37) % 61 - 20) / 256.0).astype(np.float32)
    np.testing.assert_array_equal(e, fast.gemm_i8_mul2_clamp(a, b_nk.T, scale, bool(act)))


def test_profiler_gemm_splitk_int8(tmp_path):
    """profile_gemm_splitk's argument list (KBatch = arg14); PassThrough int8 output keeps the low byte."""
    M, N, K = 128, 512, 4096
    out, dump = _run("ckx_profiler", ["gemm_splitk", 3, 1, 1, 1, 0, 1, M, N, K, -1, -1, -1, 4], "CKX_PROFILER_DUMP",
                     tmp_path)
    assert "Best Perf:" in out and "Error" not in out and "SplitK" in out
    c = np.fromfile(dump, np.int8).reshape(M, N)
    a = uniform_int8((M, K), -5, 5, SEED)
    b_nk = uniform_int8((N, K), -5, 5, SEED + 1)
    np.testing.assert_array_equal(c, fast.gemm_i8(a, b_nk.T))


def test_profiler_batched_gemm_fp16(tmp_path):
    """profile_batched_gemm's argument list (BatchCount = arg14), dense batch strides."""
    M, N, K, G = 192, 320, 256, 5
    out, dump = _run("ckx_profiler", ["batched_gemm", 1, 1, 1, 2, 0, 1, M, N, K, -1, -1, -1, G], "CKX_PROFILER_DUMP",
                     tmp_path)
    assert "Best Perf:" in out and "Error" not in out and "Batched" in out
    c = np.fromfile(dump, np.float16).reshape(G, M, N)
    a = uniform_f16((G, M, K), -1, 1, SEED)
    b_gnk = uniform_f16((G, N, K), -1, 1, SEED + 1)
    ref = lit.batched_gemm_f16(a, np.ascontiguousarray(b_gnk.transpose(0, 2, 1)))
    bad, max_err = lit.check_err_f16(c, ref, 1e-2, 1e-2)
    assert bad == 0, max_err


def test_profiler_bf16_gemm(tmp_path):
    """data type 2 of the reference profiler's gemm operation (bf16)."""
    from composable_kernel_amd.host_tensor import uniform_bf16
    M, N, K = 384, 512, 768
    out, dump = _run("ckx_profiler", ["gemm", 2, 1, 1, 2, 0, 1, M, N, K, -1, -1, -1], "CKX_PROFILER_DUMP", tmp_path)
    assert "Best Perf:" in out and "Error" not in out and "bf16" in out
    c = fast.bf16_to_f32(np.fromfile(dump, np.uint16).reshape(M, N))
    a = uniform_bf16((M, K), -1, 1, SEED)
    b_nk = uniform_bf16((N, K), -1, 1, SEED + 1)
    ref = fast.bf16_to_f32(lit.gemm_bf16(a, np.ascontiguousarray(b_nk.T)))
    assert np.all(np.abs(c - ref) <= 1e-2 + 1e-2 * np.abs(ref))


@pytest.mark.parametrize("layout", [0, 2, 3])     # mk_kn, km_kn, km_nk (profiler/src/profile_gemm.cpp:13-19)
def test_profiler_gemm_other_layouts(tmp_path, layout):
    """The layouts with a K-major operand through the C++ operator templates: A stored [K,M] for km, B stored
    [K,N] for kn, the generators filling the stored arrays in order."""
    M, N, K = 384, 512, 640
    out, dump = _run("ckx_profiler", ["gemm", 3, layout, 1, 1, 0, 1, M, N, K, -1, -1, -1, 2, 0.05, 0.4],
                     "CKX_PROFILER_DUMP", tmp_path)
    assert "Best Perf:" in out and "Error" not in out
    assert out.count("does not support this problem") >= 8      # skinny and few-row tile instances
    a_st = uniform_int8((K, M) if layout >= 2 else (M, K), -5, 5, SEED)
    b_st = uniform_int8((K, N) if layout in (0, 2) else (N, K), -5, 5, SEED + 1)
    a_mk = a_st.T if layout >= 2 else a_st
    b_kn = b_st if layout in (0, 2) else b_st.T
    c = np.fromfile(dump, np.int8).reshape(M, N)
    np.testing.assert_array_equal(c, lit.gemm_i8(a_mk, b_kn, lit.EPI_REQUANT_RND, 0.05, 0.4))
    out, dump = _run("ckx_profiler", ["gemm", 1, layout, 1, 2, 0, 1, M, N, K, -1, -1, -1], "CKX_PROFILER_DUMP", tmp_path)
    assert "Best Perf:" in out and "Error" not in out
    a_st = uniform_f16((K, M) if layout >= 2 else (M, K), -1, 1, SEED)
    b_st = uniform_f16((K, N) if layout in (0, 2) else (N, K), -1, 1, SEED + 1)
    c = np.fromfile(dump, np.float16).reshape(M, N)
    bad, max_err = lit.check_err_f16(c, lit.gemm_f16(a_st.T if layout >= 2 else a_st, b_st if layout in (0, 2) else b_st.T),
                                     1e-2, 1e-2)
    assert bad == 0, max_err


@pytest.mark.parametrize("mask", [0, 1])
def test_profiler_batched_gemm_softmax_gemm(tmp_path, mask):
    M, N, K, O, G = 256, 384, 64, 64, 3
    out, dump = _run("ckx_profiler", ["batched_gemm_softmax_gemm", 1, 1, 0, 1, M, N, K, O, G, 0.125, mask],
                     "CKX_PROFILER_DUMP", tmp_path)
    assert "Best Perf:" in out and "Error" not in out and "SoftmaxGemm" in out
    a = uniform_f16((G, M, K), -1, 1, SEED + 7)
    b0 = uniform_f16((G, N, K), -1, 1, SEED + 8)
    b1 = uniform_f16((G, N, O), -1, 1, SEED + 9)
    c = np.fromfile(dump, np.float16).reshape(G, M, O)
    want = lit.batched_gemm_softmax_gemm_f16(a, b0.transpose(0, 2, 1), b1, 0.125, bool(mask))
    bad, max_err = lit.check_err_f16(c, want, 1e-2, 1e-2)
    assert bad == 0, max_err
