"""Pins the CPU oracle (oracle/) before anything is compared against it.

Sources of truth, none of which is the oracle's own formula retyped:
  * golden vectors the reference's own tests hold (tests/golden/*.json),
  * the reference's host operators compiled in place (oracle/_ref) when built,
  * closed forms, exact rational arithmetic, and brute force on tiny inputs.
"""
import json
import os

import numpy as np
import pytest

import oracle
from composable_kernel_amd.host_tensor import uniform_f16
from oracle import lit, fast

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = json.load(open(os.path.join(HERE, "golden", "reference_conv_fwd_vectors.json")))
REF = oracle.load_ref()
needs_ref = pytest.mark.skipif(REF is None, reason="oracle/_ref not built")


# ----------------------------------------------------------------- conv golden
@pytest.mark.parametrize("case", GOLD["cases"])
def test_conv2d_reference_golden_vectors(case):
    N, K, C = case["N"], case["K"], case["C"]
    Hi, Wi = case["input"]
    Y, X = case["filter"]
    inp = np.arange(N * Hi * Wi * C, dtype=np.float32).reshape(N, Hi, Wi, C)
    wei = np.full((K, Y, X, C), 0.5, np.float32)
    out = lit.conv2d_fwd(inp, wei, case["strides"], case["dilations"], case["left_pads"],
                         case["right_pads"])
    n, k, ho, wo = case["out_dims_nkhw"]
    assert out.shape == (n, ho, wo, k)
    np.testing.assert_array_equal(out.ravel(), np.array(case["expected"], np.float32))
    # the numpy im2col form must agree as well (fp32 exact here: small integers and halves)
    cols, Ho, Wo = fast.im2col(inp, Y, X, case["strides"], case["dilations"], case["left_pads"],
                               case["right_pads"])
    np.testing.assert_array_equal((cols @ wei.reshape(K, -1).T).ravel(),
                                  np.array(case["expected"], np.float32))
    if REF is not None:
        np.testing.assert_array_equal(
            REF.conv2d_fwd(inp, wei, case["strides"], case["dilations"], case["left_pads"]), out)


def test_conv_out_len_known_answers():
    for c in GOLD["conv_out_len_known_answers"]["cases"]:
        assert lit.conv_out_len(c["in"], c["filter"], c["stride"], c["dilation"], c["pad_l"],
                                c["pad_r"]) == c["out"]
        if REF is not None:
            assert REF.conv_out_len(c["in"], c["filter"], c["stride"], c["dilation"], c["pad_l"],
                                    c["pad_r"]) == c["out"]


# -------------------------------------------------------------- magic division
def test_magic_division_matches_integer_division():
    # same sweep as test/magic_number_division/magic_number_division.cpp:59-138
    rng = np.random.default_rng(1)
    dividends = np.concatenate([np.arange(0, 5000), rng.integers(0, 2 ** 31 - 1, 3000),
                                [2 ** 31 - 1, 2 ** 31 - 2, 2 ** 30]]).astype(np.uint64)
    for d in list(range(1, 4097)) + [65535, 65536, 802816, 2 ** 31 - 1]:
        m, s = lit.magic_params(d)
        q = ((dividends * np.uint64(m)) >> np.uint64(32)) + dividends
        q = (q & np.uint64(0xFFFFFFFF)) >> np.uint64(s)
        np.testing.assert_array_equal(q, dividends // np.uint64(d), err_msg=f"divisor {d}")
    for d in (1, 3, 7, 56, 576, 4096):
        m, s = lit.magic_params(d)
        for n in (0, 1, d - 1, d, d + 1, 123456789, 2 ** 31 - 1):
            assert lit.magic_divide(n, m, s) == n // d
        if REF is not None:
            assert REF.magic_params(d) == (m, s)


# ------------------------------------------------------------ fp16 conversions
def test_half_conversions_match_ieee():
    L = lit.lib()
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    got = np.array([L.cko_half_to_float(int(h)) for h in allh], np.float32)
    fin = np.isfinite(want)
    np.testing.assert_array_equal(got[fin], want[fin])
    assert np.all(np.isnan(got[np.isnan(want)]))
    np.testing.assert_array_equal(got[np.isinf(want)], want[np.isinf(want)])
    rng = np.random.default_rng(2)
    f = np.concatenate([
        rng.uniform(-70000, 70000, 4000), rng.uniform(-1, 1, 4000), rng.uniform(-1e-4, 1e-4, 4000),
        rng.uniform(-1e-7, 1e-7, 2000),
        # exact ties between neighbouring halves
        (allh[1:30000:7].view(np.float16).astype(np.float64)
         + allh[2:30001:7].view(np.float16).astype(np.float64)) / 2,
        [65504, 65519.99, 65520, 65536, 5.9604645e-08, 2.9802322e-08, 2.98023224e-08 * 1.0000001, 0.0]
    ]).astype(np.float32)
    want16 = f.astype(np.float16).view(np.uint16)
    got16 = np.array([L.cko_float_to_half(float(x)) for x in f], np.uint16)
    np.testing.assert_array_equal(got16, want16)


# ------------------------------------------------------------------- epilogue
def _epilogue_exact(acc, epi, sg, sr):
    """Independent derivation: a float32 x float32 product is exact in float64, so one
    float64 multiply followed by one rounding to float32 equals the IEEE fp32 multiply."""
    if epi == lit.EPI_PASSTHROUGH:
        return ((acc + 128) % 256) - 128
    sg, sr = np.float32(sg), np.float32(sr)
    x = np.float32(acc)
    assert float(x) == acc
    g = np.float32(np.float64(sg) * np.float64(x))
    if epi == lit.EPI_REQUANT_CK:
        r = g if g > 0 else np.float32(0)
        q = np.float32(np.float64(sr) * np.float64(r))
        y = min(max(float(q), -128.0), 127.0)
        return int(y)  # toward zero
    t = float(round(float(g)))  # Python round() is half-to-even on an exact binary value
    t = min(max(t, -128.0), 127.0)
    r = max(t, 0.0)
    u = float(round(float(np.float32(np.float64(sr) * np.float64(np.float32(r))))))
    return int(min(max(u, -128.0), 127.0))


@pytest.mark.parametrize("epi,sg,sr", [
    (lit.EPI_REQUANT_CK, 0.03, 1.0), (lit.EPI_REQUANT_RND, 0.5, 0.03), (lit.EPI_REQUANT_RND, 0.02, 0.4),
    (lit.EPI_REQUANT_CK, 0.5, 0.03), (lit.EPI_REQUANT_RND, 0.03, 1.0), (lit.EPI_PASSTHROUGH, 1.0, 1.0),
])
def test_epilogue_scalar_against_exact_arithmetic(epi, sg, sr):
    rng = np.random.default_rng(3)
    accs = list(range(-700, 9000)) + [int(v) for v in rng.integers(-2 ** 20, 2 ** 20, 4000)] + \
        [2 ** 24 - 1, -(2 ** 24 - 1), 704512, -704512]
    for acc in accs:
        assert lit.epilogue_i8(acc, epi, sg, sr) == _epilogue_exact(acc, epi, sg, sr), (acc, epi)
    arr = np.array(accs, np.int32)
    np.testing.assert_array_equal(fast.epilogue_i8(arr, epi, sg, sr),
                                  np.array([lit.epilogue_i8(a, epi, sg, sr) for a in accs], np.int8))


def _mul2_clamp_exact(acc, scale, relu):
    """Independent derivation of Activation_Mul2_Clamp: exact fp32 product through float64 (as above), ordinary
    min / max, truncation toward zero."""
    x = np.float32(acc)
    if relu and x < 0:
        x = np.float32(0)
    y = np.float32(np.float64(np.float32(scale)) * np.float64(x))
    return int(min(max(float(y), -128.0), 127.0))


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("scale", [0.03, -0.03, 0.4, 1.0, 2.0 ** -20, 37.5, 0.0, -1.0])
def test_mul2_clamp_scalar_against_exact_arithmetic(scale, relu):
    """The per-channel functor (upstream's Activation_Mul2_Clamp; absent from the reference snapshot, so no reference
    vectors: parity unpinned by the reference, pinned by what follows)."""
    rng = np.random.default_rng(4)
    accs = list(range(-5000, 5000)) + [int(v) for v in rng.integers(-2 ** 24, 2 ** 24, 4000)] + \
        [2 ** 24, -(2 ** 24), 2 ** 24 + 1, 2 ** 31 - 1, -(2 ** 31)]       # beyond 2^24 the conversion itself rounds
    for acc in accs:
        assert lit.mul2_clamp(acc, scale, relu) == _mul2_clamp_exact(acc, scale, relu), (acc, scale, relu)
    arr = np.array(accs, np.int32)
    np.testing.assert_array_equal(fast.epilogue_i8_mul2_clamp(arr, np.float32(scale), relu),
                                  np.array([lit.mul2_clamp(a, scale, relu) for a in accs], np.int8))


def test_mul2_clamp_closed_forms():
    # the Relu form with requant scale s IS the reference's RequantReluRequant(1, s), literal form (example 14):
    # both are trunc(clamp(s * relu(float(acc)))) -- and that functor is pinned against the reference itself
    for s in (0.03, 0.4, 1.0, 2.5, 0.0078125):
        for acc in list(range(-300, 6000, 7)) + [10 ** 6, -10 ** 6]:
            assert lit.mul2_clamp(acc, s, True) == lit.epilogue_i8(acc, lit.EPI_REQUANT_CK, 1.0, s)
    # dyadic scales: the product is exact, the result is integer arithmetic -- truncation TOWARD ZERO on both sides
    for k in (1, 3, 100, 255):
        for acc in range(-2000, 2000):
            q = acc * k                      # value * 256
            want = max(-128, min(127, -((-q) // 256) if q < 0 else q // 256))
            assert lit.mul2_clamp(acc, k / 256.0, False) == want
    # clamp is asymmetric, a negative scale flips the sign after the ReLU, zero scale gives zero
    assert lit.mul2_clamp(10 ** 6, 1.0, False) == 127 and lit.mul2_clamp(-10 ** 6, 1.0, False) == -128
    assert lit.mul2_clamp(100, -0.5, True) == -50 and lit.mul2_clamp(-100, -0.5, True) == 0
    assert lit.mul2_clamp(-100, -0.5, False) == 50 and lit.mul2_clamp(12345, 0.0, False) == 0
    # per column: column n of the GEMM form uses scale n only
    a = np.arange(-20, 20, dtype=np.int8).reshape(5, 8)
    b = (np.arange(24, dtype=np.int8).reshape(8, 3) - 11)
    s = np.array([0.5, -0.25, 3.0], np.float32)
    acc = a.astype(np.int64) @ b.astype(np.int64)
    for relu in (False, True):
        out = lit.gemm_i8_mul2_clamp(a, b, s, relu)
        np.testing.assert_array_equal(out, fast.gemm_i8_mul2_clamp(a, b, s, relu))
        for n in range(3):
            assert [int(v) for v in out[:, n]] == [_mul2_clamp_exact(int(v), s[n], relu) for v in acc[:, n]]


def test_epilogue_special_cases():
    R, Cc = lit.EPI_REQUANT_RND, lit.EPI_REQUANT_CK
    # ties go to even with scale 0.5
    assert [lit.epilogue_i8(a, R, 0.5, 1.0) for a in (1, 3, 5, 7, 2, 254, 255, 256, 1000)] == \
        [0, 2, 2, 4, 1, 127, 127, 127, 127]
    # negative accumulators die in the ReLU
    assert all(lit.epilogue_i8(a, m, 0.5, 0.03) == 0 for a in (-1, -77, -10 ** 6) for m in (R, Cc))
    # literal functor truncates toward zero instead of rounding: 0.03*66 = 1.98 -> 1
    assert lit.epilogue_i8(66, Cc, 0.03, 1.0) == 1
    assert lit.epilogue_i8(66, R, 0.03, 1.0) == 2
    assert lit.epilogue_i8(10 ** 6, Cc, 0.03, 1.0) == 127
    # inner saturation is visible in the rounded mode: 0.5*400=200 -> 127 -> *0.5 = 63.5 -> 64
    assert lit.epilogue_i8(400, R, 0.5, 0.5) == 64
    # passthrough keeps the low byte
    assert [lit.epilogue_i8(a, lit.EPI_PASSTHROUGH, 1, 1) for a in (14400, -300, 255, 128)] == \
        [64, -44, -1, -128]


# ----------------------------------------------------------------------- GEMM
def _rand_i8(rng, shape, lo=-5, hi=5):
    return rng.integers(lo, hi + 1, shape).astype(np.int8)


def test_gemm_i8_closed_forms():
    M, N, K = 7, 9, 40
    ones_a, ones_b = np.ones((M, K), np.int8), np.ones((K, N), np.int8)
    np.testing.assert_array_equal(lit.gemm_i8_acc(ones_a, ones_b), np.full((M, N), K, np.int32))
    a = np.repeat(np.arange(M, dtype=np.int8)[:, None], K, 1)   # A(m,k) = m
    b = np.repeat(np.arange(N, dtype=np.int8)[None, :], K, 0)   # B(k,n) = n
    want = K * np.arange(M)[:, None] * np.arange(N)[None, :]
    np.testing.assert_array_equal(lit.gemm_i8_acc(a, b), want)
    # int32 accumulate + PassThrough keeps the low byte; float accumulate agrees
    np.testing.assert_array_equal(lit.gemm_i8(a, b), (want & 0xFF).astype(np.uint8).view(np.int8))
    np.testing.assert_array_equal(lit.gemm_i8(a, b, acc_float=True),
                                  (want & 0xFF).astype(np.uint8).view(np.int8))
    # identity B
    rng = np.random.default_rng(4)
    a = _rand_i8(rng, (5, 6), -128, 127)
    np.testing.assert_array_equal(lit.gemm_i8(a, np.eye(6, dtype=np.int8)), a)


def test_gemm_i8_brute_force_and_layouts():
    rng = np.random.default_rng(5)
    M, N, K = 6, 5, 33
    a = _rand_i8(rng, (M, K), -128, 127)
    b_nk = _rand_i8(rng, (N, K), -128, 127)          # column-major B: K contiguous
    want = np.zeros((M, N), np.int64)
    for m in range(M):
        for n in range(N):
            for k in range(K):
                want[m, n] += int(a[m, k]) * int(b_nk[n, k])
    np.testing.assert_array_equal(lit.gemm_i8_acc(a, b_nk.T), want)
    # row-major B gives the same through different strides
    np.testing.assert_array_equal(lit.gemm_i8_acc(a, np.ascontiguousarray(b_nk.T)), want)
    # column-major A
    np.testing.assert_array_equal(lit.gemm_i8_acc(np.asfortranarray(a), b_nk.T), want)
    # transposition symmetry C(A,B)^T = C(B^T, A^T)
    np.testing.assert_array_equal(lit.gemm_i8_acc(b_nk, a.T), want.T)


@pytest.mark.parametrize("epi,sg,sr", [(lit.EPI_REQUANT_CK, 0.03, 1.0), (lit.EPI_REQUANT_RND, 0.5, 0.03),
                                       (lit.EPI_REQUANT_RND, 0.02, 0.4), (lit.EPI_PASSTHROUGH, 1, 1)])
def test_gemm_i8_lit_fast_ref_agree(epi, sg, sr):
    rng = np.random.default_rng(6)
    for (M, N, K, lo, hi) in [(64, 48, 80, -5, 5), (33, 17, 1024, -8, 8), (1, 130, 256, -5, 5)]:
        a = _rand_i8(rng, (M, K), lo, hi)
        b_nk = _rand_i8(rng, (N, K), lo, hi)
        c_lit = lit.gemm_i8(a, b_nk.T, epi, sg, sr)
        np.testing.assert_array_equal(fast.gemm_i8(a, b_nk.T, epi, sg, sr), c_lit)
        # epilogue of the exact accumulators, element by element, through the exact-arithmetic form
        acc = lit.gemm_i8_acc(a, b_nk.T)
        idx = rng.integers(0, acc.size, 200)
        for i in idx:
            assert c_lit.ravel()[i] == _epilogue_exact(int(acc.ravel()[i]), epi, sg, sr)
        if REF is not None:
            if epi == lit.EPI_PASSTHROUGH:
                np.testing.assert_array_equal(REF.gemm_i8(a, b_nk.T), c_lit)
            else:
                np.testing.assert_array_equal(REF.gemm_i8_requant(a, b_nk.T, epi, sg, sr), c_lit)


def test_gemm_i8_thread_count_is_unobservable():
    rng = np.random.default_rng(7)
    a, b = _rand_i8(rng, (37, 64)), _rand_i8(rng, (64, 29))
    c1 = lit.gemm_i8(a, b, lit.EPI_REQUANT_RND, 0.5, 0.03, nthreads=1)
    for t in (2, 3, 8, 64):
        np.testing.assert_array_equal(lit.gemm_i8(a, b, lit.EPI_REQUANT_RND, 0.5, 0.03, nthreads=t), c1)


def test_gemm_f16_against_float64_and_ref():
    rng = np.random.default_rng(8)
    M, N, K = 24, 40, 96
    a = rng.uniform(-1, 1, (M, K)).astype(np.float16)
    b_nk = rng.uniform(-1, 1, (N, K)).astype(np.float16)
    c = lit.gemm_f16(a, b_nk.T)
    # sequential fp32 summation restated independently with numpy scalars
    want = np.zeros((M, N), np.float16)
    for m in range(M):
        for n in range(N):
            acc = np.float32(0)
            for k in range(K):
                acc = np.float32(acc + np.float32(a[m, k]) * np.float32(b_nk[n, k]))
            want[m, n] = np.float16(acc)
    np.testing.assert_array_equal(c.view(np.uint16), want.view(np.uint16))
    exact = a.astype(np.float64) @ b_nk.T.astype(np.float64)
    assert np.max(np.abs(c.astype(np.float64) - exact)) < 2e-2
    bad, _ = lit.check_err_f16(fast.gemm_f16(a, b_nk.T), c, 1e-3, 1e-3)
    assert bad == 0
    if REF is not None:
        np.testing.assert_array_equal(REF.gemm_f16(a, b_nk.T).view(np.uint16), c.view(np.uint16))
    # closed form: all ones -> K (exact in fp16 for K <= 2048)
    np.testing.assert_array_equal(lit.gemm_f16(np.ones((3, 512), np.float16), np.ones((512, 4), np.float16)),
                                  np.full((3, 4), 512, np.float16))


def test_batched_gemm_and_gemm_gemm():
    rng = np.random.default_rng(9)
    G, M, K, N, O = 3, 10, 16, 12, 8
    a = rng.uniform(-0.5, 0.5, (G, M, K)).astype(np.float16)
    b0_gnk = rng.uniform(-0.5, 0.5, (G, N, K)).astype(np.float16)   # column-major K x N per batch
    b1 = rng.uniform(-0.5, 0.5, (G, N, O)).astype(np.float16)
    b0 = b0_gnk.transpose(0, 2, 1)
    s = lit.batched_gemm_f16(a, b0)
    for g in range(G):   # batch independence + equality with the plain GEMM oracle
        np.testing.assert_array_equal(s[g].view(np.uint16), lit.gemm_f16(a[g], b0[g]).view(np.uint16))
    if REF is not None:
        np.testing.assert_array_equal(REF.batched_gemm_f16(a, b0).view(np.uint16), s.view(np.uint16))
    c = lit.batched_gemm_gemm_f16(a, b0, b1)
    # brute force with an fp16 intermediate
    want = np.zeros((G, M, O), np.float16)
    for g in range(G):
        for m in range(M):
            for o in range(O):
                acc = np.float32(0)
                for n in range(N):
                    acc = np.float32(acc + np.float32(s[g, m, n]) * np.float32(b1[g, n, o]))
                want[g, m, o] = np.float16(acc)
    np.testing.assert_array_equal(c.view(np.uint16), want.view(np.uint16))
    if REF is not None:
        np.testing.assert_array_equal(REF.batched_gemm_f16(s, b1).view(np.uint16), c.view(np.uint16))
    bad, _ = lit.check_err_f16(fast.batched_gemm_gemm_f16(a, b0, b1), c, 1e-2, 1e-2)
    assert bad == 0
    # closed form: ones -> K then N*K
    one = np.ones
    np.testing.assert_array_equal(
        lit.batched_gemm_gemm_f16(one((1, 2, 4), np.float16), one((1, 4, 8), np.float16),
                                  one((1, 8, 3), np.float16)), np.full((1, 2, 3), 32, np.float16))


# ----------------------------------------------------------------------- conv
@pytest.mark.parametrize("dtype", [np.float16, np.int8])
def test_conv2d_lit_fast_ref_agree(dtype):
    rng = np.random.default_rng(10)
    for (N, C, K, Hi, Wi, Y, X, s, d, p) in [(2, 8, 16, 5, 6, 3, 3, (2, 1), (1, 2), (1, 2)),
                                             (1, 16, 4, 7, 7, 1, 1, (2, 2), (1, 1), (0, 0)),
                                             (2, 3, 5, 9, 8, 3, 2, (1, 1), (1, 1), (1, 0))]:
        if dtype == np.int8:
            inp = _rand_i8(rng, (N, Hi, Wi, C))
            wei = _rand_i8(rng, (K, Y, X, C))
        else:
            inp = rng.uniform(-1, 1, (N, Hi, Wi, C)).astype(np.float16)
            wei = rng.uniform(-1, 1, (K, Y, X, C)).astype(np.float16)
        out = lit.conv2d_fwd(inp, wei, s, d, p)
        if dtype == np.int8:
            np.testing.assert_array_equal(fast.conv2d_fwd_i8(inp, wei, s, d, p), out)
            # the requant functor as OutElementOp
            o2 = lit.conv2d_fwd(inp, wei, s, d, p, epi=lit.EPI_REQUANT_RND, scale_gemm=0.5, scale_relu=0.3)
            np.testing.assert_array_equal(
                fast.conv2d_fwd_i8(inp, wei, s, d, p, epi=lit.EPI_REQUANT_RND, scale_gemm=0.5,
                                   scale_relu=0.3), o2)
        else:
            bad, _ = lit.check_err_f16(fast.conv2d_fwd_f16(inp, wei, s, d, p), out, 1e-3, 1e-3)
            assert bad == 0
        if REF is not None:
            np.testing.assert_array_equal(REF.conv2d_fwd(inp, wei, s, d, p).view(np.uint8),
                                          out.view(np.uint8))


GOLD_ND = json.load(open(os.path.join(HERE, "golden", "reference_convnd_fwd_vectors.json")))


def _monotonic_fill(n, start, step):
    """FillMonotonicSeq (library/include/ck/library/utility/fill.hpp:66-80): x[i+1] = x[i] + step in fp32."""
    out = np.empty(n, np.float32)
    v = np.float32(start)
    for i in range(n):
        out[i] = v
        v = np.float32(v + np.float32(step))
    return out


@pytest.mark.parametrize("case", GOLD_ND["cases"], ids=lambda c: c["name"])
def test_convnd_reference_golden_vectors(case):
    """The 1-D (NWC) and 3-D (NCDHW) outputs the reference's own ReferenceConvFwd test holds
    (test/reference_conv_fwd/reference_conv_fwd.cpp:156-392), with that test's check_err tolerances."""
    N, K, C = case["N"], case["K"], case["C"]
    sp, filt = case["input"], case["filter"]
    x = _monotonic_fill(N * C * int(np.prod(sp)), *case["fill_start_step"])
    if case["layout"] == "channels_first":
        inp = np.moveaxis(x.reshape(N, C, *sp), 1, -1)
    else:
        inp = x.reshape(N, *sp, C)
    wei = np.full((K, *filt, C), 0.5, np.float32)
    out = lit.convnd_fwd(inp, wei, case["strides"], case["dilations"], case["left_pads"], case["right_pads"])
    assert list(out.shape) == [N, *case["out_dims_nk_spatial"][2:], K]
    got = (np.moveaxis(out, -1, 1) if case["layout"] == "channels_first" else out).ravel()
    exp = np.array(case["expected"], np.float32)
    assert got.shape == exp.shape
    assert (np.abs(got.astype(np.float64) - exp) <= case["atol"] + case["rtol"] * np.abs(exp)).all()
    # BLAS / im2col form (another summation order, result rounded to fp16)
    np.testing.assert_allclose(
        fast.convnd_fwd(inp, wei, case["strides"], case["dilations"], case["left_pads"],
                        case["right_pads"]).astype(np.float32), out, rtol=2e-3, atol=1e-3)
    if REF is not None:
        np.testing.assert_array_equal(
            REF.convnd_fwd(inp, wei, case["strides"], case["dilations"], case["left_pads"]), out)


@pytest.mark.parametrize("dtype", [np.float16, np.int8])
def test_convnd_lit_fast_ref_agree(dtype):
    """One and three spatial dimensions: literal restatement, im2col + BLAS form and the compiled reference."""
    rng = np.random.default_rng(11)
    for (shape_in, shape_w, s, d, p) in [((2, 9, 8), (5, 3, 8), (2,), (2,), (1,)),
                                         ((3, 11, 16), (4, 1, 16), (1,), (1,), (0,)),
                                         ((2, 5, 7, 6, 8), (5, 2, 3, 2, 8), (1, 2, 1), (2, 1, 2), (1, 1, 0)),
                                         ((1, 4, 4, 4, 16), (3, 3, 3, 3, 16), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
                                         ((2, 3, 5, 4, 8), (6, 1, 1, 1, 8), (2, 2, 2), (1, 1, 1), (0, 0, 0))]:
        if dtype == np.int8:
            inp, wei = _rand_i8(rng, shape_in), _rand_i8(rng, shape_w)
        else:
            inp = rng.uniform(-1, 1, shape_in).astype(np.float16)
            wei = rng.uniform(-1, 1, shape_w).astype(np.float16)
        out = lit.convnd_fwd(inp, wei, s, d, p)
        if dtype == np.int8:
            np.testing.assert_array_equal(fast.convnd_fwd(inp, wei, s, d, p), out)
            o2 = lit.convnd_fwd(inp, wei, s, d, p, epi=lit.EPI_REQUANT_RND, scale_gemm=0.5, scale_relu=0.3)
            np.testing.assert_array_equal(
                fast.convnd_fwd(inp, wei, s, d, p, epi=lit.EPI_REQUANT_RND, scale_gemm=0.5, scale_relu=0.3), o2)
        else:
            bad, _ = lit.check_err_f16(fast.convnd_fwd(inp, wei, s, d, p), out, 1e-3, 1e-3)
            assert bad == 0
        if REF is not None:
            np.testing.assert_array_equal(REF.convnd_fwd(inp, wei, s, d, p).view(np.uint8), out.view(np.uint8))
    # two dimensions through the N-d entry are the 2-D routine
    inp, wei = _rand_i8(rng, (2, 6, 7, 8)), _rand_i8(rng, (4, 3, 2, 8))
    np.testing.assert_array_equal(lit.convnd_fwd(inp, wei, (1, 2), (2, 1), (1, 1)),
                                  lit.conv2d_fwd(inp, wei, (1, 2), (2, 1), (1, 1)))


def test_conv2d_int8_passthrough_wraps_modulo_256():
    # the reference's int8 conv keeps the low byte of an out-of-range sum
    inp = np.full((1, 4, 4, 16), 5, np.int8)
    wei = np.full((2, 3, 3, 16), 5, np.int8)
    out = lit.conv2d_fwd(inp, wei, pads=(0, 0))
    assert out.shape == (1, 2, 2, 2)
    total = 25 * 9 * 16   # 3600
    assert int(out[0, 0, 0, 0]) == ((total + 128) % 256) - 128


def test_conv2d_is_a_gemm_for_1x1():
    rng = np.random.default_rng(11)
    inp = _rand_i8(rng, (2, 4, 5, 32))
    wei = _rand_i8(rng, (8, 1, 1, 32))
    out = lit.conv2d_fwd(inp, wei)
    np.testing.assert_array_equal(out.reshape(-1, 8), lit.gemm_i8(inp.reshape(-1, 32), wei.reshape(8, 32).T))


# ------------------------------------------------- fused bias / ReLU / residual epilogues
@pytest.mark.parametrize("case", [c for c in GOLD["cases"] if max(c["expected"]) < 2000 and
                                  c["left_pads"] == c["right_pads"]])
def test_conv2d_bias_relu_on_the_reference_golden_vectors(case):
    """The reference's golden conv outputs (all exactly representable in fp16 for these cases)
    pushed through AddRelu / AddReluAdd by hand: the bias is chosen so that ReLU cuts part of the
    outputs, the residual is negative so that relu(acc + b) + r differs from relu(acc + b + r)."""
    N, K, C = case["N"], case["K"], case["C"]
    Hi, Wi = case["input"]
    Y, X = case["filter"]
    inp = np.arange(N * Hi * Wi * C, dtype=np.float32).reshape(N, Hi, Wi, C).astype(np.float16)
    wei = np.full((K, Y, X, C), 0.5, np.float16)
    gold = np.array(case["expected"], np.float32)
    n, k, ho, wo = case["out_dims_nkhw"]
    gold = gold.reshape(n, ho, wo, k)
    assert np.array_equal(gold.astype(np.float16).astype(np.float32), gold)
    bias = (-np.median(gold) - 0.5 * np.arange(K)).astype(np.float16)
    resi = np.full(gold.shape, -3.0, np.float16)
    want = np.maximum(gold + bias.astype(np.float32), 0)
    out = lit.conv2d_fwd_bias_relu_f16(inp, wei, bias, None, case["strides"], case["dilations"], case["left_pads"])
    np.testing.assert_array_equal(out, want.astype(np.float16))
    assert (out == 0).any() and (out > 0).any()
    out2 = lit.conv2d_fwd_bias_relu_f16(inp, wei, bias, resi, case["strides"], case["dilations"], case["left_pads"])
    np.testing.assert_array_equal(out2, (want - 3.0).astype(np.float16))
    assert (out2 == -3).any()
    np.testing.assert_array_equal(
        fast.conv2d_fwd_bias_relu_f16(inp, wei, bias, resi, case["strides"], case["dilations"], case["left_pads"]), out2)
    if REF is not None:
        np.testing.assert_array_equal(
            REF.conv2d_fwd_bias_relu_f16(inp, wei, bias, None, case["strides"], case["dilations"], case["left_pads"]), out)
        np.testing.assert_array_equal(
            REF.conv2d_fwd_bias_relu_f16(inp, wei, bias, resi, case["strides"], case["dilations"], case["left_pads"]), out2)


def test_conv2d_bias_relu_random_lit_fast_ref_agree():
    rng = np.random.default_rng(5)
    inp = rng.uniform(-1, 1, (2, 9, 7, 8)).astype(np.float16)
    wei = rng.uniform(-1, 1, (5, 3, 3, 8)).astype(np.float16)
    bias = rng.uniform(-2, 2, 5).astype(np.float16)
    out_shape = (2, 5, 4, 5)
    resi = rng.uniform(-2, 2, out_shape).astype(np.float16)
    for r in (None, resi):
        a = lit.conv2d_fwd_bias_relu_f16(inp, wei, bias, r, (2, 2), (1, 1), (1, 1))
        assert a.shape == out_shape
        b = fast.conv2d_fwd_bias_relu_f16(inp, wei, bias, r, (2, 2), (1, 1), (1, 1))
        assert np.all(np.abs(a.astype(np.float32) - b.astype(np.float32)) <= 2e-3 + 2e-3 * np.abs(b.astype(np.float32)))
        if REF is not None:
            np.testing.assert_array_equal(REF.conv2d_fwd_bias_relu_f16(inp, wei, bias, r, (2, 2), (1, 1), (1, 1)), a)


def test_gemm_add_relu_rounds_c_to_fp16_before_the_functor():
    """Example 03 hands the fp32 GEMM result to a functor on half_t operands: C is rounded first.
    K = 2049 ones give acc = 2049, fp16 2048 (tie to even); + 1 = 2049 -> 2048 again. A single
    rounding of acc + d = 2050 would give 2050. Negative sums must come out as +0."""
    a = np.ones((3, 2049), np.float16)
    b = np.ones((2049, 4), np.float16)
    d = np.array([1.0, -1.0, -4096.0, 0.0], np.float16)[None, :]
    e = lit.gemm_f16_add_relu(a, b, d)
    np.testing.assert_array_equal(e, np.broadcast_to(np.array([2048, 2047, 0, 2048], np.float16), (3, 4)))
    assert not np.signbit(e).any()
    np.testing.assert_array_equal(fast.gemm_f16_add_relu(a, b, d), e)
    if REF is not None:
        np.testing.assert_array_equal(REF.gemm_f16_add_relu(a, b, d), e)


def test_gemm_add_relu_random_lit_ref_bit_exact_and_full_d():
    rng = np.random.default_rng(8)
    a = rng.uniform(-1, 1, (17, 96)).astype(np.float16)
    b = np.asfortranarray(rng.uniform(-1, 1, (96, 23)).astype(np.float16))
    for d in (rng.uniform(-3, 3, (1, 23)).astype(np.float16), rng.uniform(-3, 3, (17, 23)).astype(np.float16)):
        e = lit.gemm_f16_add_relu(a, b, d)
        c = lit.gemm_f16(a, b)
        x = (c.astype(np.float32) + np.broadcast_to(d, c.shape).astype(np.float32)).astype(np.float16)
        np.testing.assert_array_equal(e, np.maximum(x, np.float16(0)))
        if REF is not None:
            np.testing.assert_array_equal(REF.gemm_f16_add_relu(a, b, d), e)


# ------------------------------------------------------------------- Bilinear / AddAddFastGelu
def test_gemm_bilinear_rounds_once_and_reduces_to_its_parts():
    """alpha * acc + beta * d is rounded ONCE: K = 2049 ones give acc = 2049; + 1 = 2050 is a fp16 value (rounding C
    first would store 2048). alpha = 1, beta = 0 is the plain GEMM; alpha = 0, beta = 1 returns D bit for bit;
    small integers are exact. The reference's own functor agrees bit for bit."""
    a = np.ones((3, 2049), np.float16)
    b = np.ones((2049, 4), np.float16)
    d = np.array([1.0, -1.0, -4096.0, 0.5], np.float16)[None, :]
    e = lit.gemm_f16_bilinear(a, b, d, 1.0, 1.0)
    np.testing.assert_array_equal(e, np.broadcast_to(np.array([2050, 2048, -2047, 2050], np.float16), (3, 4)))
    np.testing.assert_array_equal(lit.gemm_f16_bilinear(a, b, d, 2.0, -3.0),
                                  np.broadcast_to(np.array([4095, 4100, 16384, 4096], np.float16), (3, 4)))
    rng = np.random.default_rng(21)
    a = rng.uniform(-1, 1, (19, 72)).astype(np.float16)
    b = np.asfortranarray(rng.uniform(-1, 1, (72, 13)).astype(np.float16))
    d = rng.uniform(-3, 3, (19, 13)).astype(np.float16)
    np.testing.assert_array_equal(lit.gemm_f16_bilinear(a, b, d, 1.0, 0.0), lit.gemm_f16(a, b))
    np.testing.assert_array_equal(lit.gemm_f16_bilinear(a, b, d, 0.0, 1.0), d)
    e = lit.gemm_f16_bilinear(a, b, d, 0.75, -1.5)
    assert lit.check_err_f16(fast.gemm_f16_bilinear(a, b, d, 0.75, -1.5), e, 1e-3, 1e-3)[0] == 0
    # swapped scalars or operands change the result
    assert (lit.gemm_f16_bilinear(a, b, d, -1.5, 0.75) != e).mean() > 0.9
    if REF is not None:
        np.testing.assert_array_equal(REF.gemm_f16_bilinear(a, b, d, 0.75, -1.5), e)
        np.testing.assert_array_equal(REF.gemm_f16_bilinear(a, b, d[:1], 0.75, -1.5),
                                      lit.gemm_f16_bilinear(a, b, d[:1], 0.75, -1.5))


def test_fast_gelu_against_the_tanh_form_and_its_limits():
    """fast_gelu(x) = 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) with the constants rounded to six digits
    (0.035677 = 0.044715 * 0.797885): checked against the tanh form in float64, at 0, and far out on both sides,
    where it is x and -0 / 0 (no NaN from the overflowing exponential)."""
    xs = np.concatenate([np.linspace(-12, 12, 481), [1e-3, -1e-3, 30.0, -30.0, 65504.0, -65504.0]])
    for x in xs:
        want = 0.5 * x * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x ** 3)))
        got = lit.fast_gelu(x)
        assert np.isfinite(got)
        assert abs(got - want) <= 2e-6 * max(1.0, abs(x)), (x, got, want)
    assert lit.fast_gelu(0.0) == 0.0
    assert lit.fast_gelu(40.0) == 40.0 and lit.fast_gelu(-40.0) == 0.0
    assert lit.fast_gelu(-0.5) < 0 < lit.fast_gelu(0.5)
    np.testing.assert_allclose(fast.fast_gelu(xs.astype(np.float32)), [lit.fast_gelu(x) for x in xs],
                               rtol=2e-6, atol=1e-7)
    if REF is not None:
        for x in xs:
            assert abs(REF.fast_gelu(x) - lit.fast_gelu(x)) <= 1e-6 * max(1.0, abs(x))


def test_gemm_add_add_fastgelu_lit_fast_ref():
    """example 04's layout: D0 a bias row (stride 0), D1 a full tensor. The literal form against the reference's own
    functor (bit-exact up to the exp of the C library in use: at most one fp16 ulp on a handful of elements) and the
    BLAS form; with A = 0 it is fast_gelu(d0 + d1) element by element; D0 and D1 are interchangeable."""
    rng = np.random.default_rng(22)
    a = rng.uniform(-1, 1, (21, 64)).astype(np.float16)
    b = np.asfortranarray(rng.uniform(-1, 1, (64, 18)).astype(np.float16))
    d0 = rng.uniform(-3, 3, (1, 18)).astype(np.float16)
    d1 = rng.uniform(-2, 2, (21, 18)).astype(np.float16)
    e = lit.gemm_f16_add_add_fastgelu(a, b, d0, d1)
    assert (e < 0).any() and (e > 1).any()
    assert lit.check_err_f16(fast.gemm_f16_add_add_fastgelu(a, b, d0, d1), e, 1e-3, 1e-3)[0] == 0
    z = lit.gemm_f16_add_add_fastgelu(np.zeros_like(a), b, d0, d1)
    s = np.broadcast_to(d0, d1.shape).astype(np.float32) + d1.astype(np.float32)
    want = np.array([lit.fast_gelu(v) for v in s.ravel()], np.float32).astype(np.float16).reshape(s.shape)
    np.testing.assert_array_equal(z, want)
    d0_full = np.ascontiguousarray(np.broadcast_to(d0, d1.shape))
    np.testing.assert_array_equal(lit.gemm_f16_add_add_fastgelu(a, b, d1, d0_full), e)
    if REF is not None:
        r = REF.gemm_f16_add_add_fastgelu(a, b, d0, d1)
        ulp = np.abs(r.view(np.int16).astype(np.int32) - e.view(np.int16).astype(np.int32))
        assert ulp.max() <= 1 and (ulp != 0).mean() < 0.02


# ------------------------------------------------------------------------------- bfloat16
def test_bf16_conversion_is_round_to_nearest_even_like_torch_and_the_reference():
    """type_convert<bhalf_t, float> (data_type.hpp:953-993): checked against torch's bfloat16 cast (an
    independent RNE implementation) on random floats, exact ties, the largest finite values and
    subnormals, and against the reference's own function."""
    import torch
    rng = np.random.default_rng(11)
    x = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 4000).astype(np.float32),
        np.array([1.0, 1.00390625, 1.01171875, 1.0078125, -1.00390625, 3.3895314e38, 3.4028235e38, 1e-40, -1e-45, 0.0,
                  -0.0, 65280.0, 65408.0], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = lit.float_to_bf16(x)
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(fast.f32_to_bf16(x), want)
    # ties: 1 + 2^-8 is halfway between bf16(1.0) = 0x3F80 and 0x3F81 -> even (0x3F80); 1 + 3*2^-8 -> 0x3F82
    assert lit.float_to_bf16(np.float32(1.00390625)) == 0x3F80 and lit.float_to_bf16(np.float32(1.01171875)) == 0x3F82
    np.testing.assert_array_equal(fast.bf16_to_f32(got), torch.from_numpy(x).to(torch.bfloat16).float().numpy())
    if REF is not None:
        for v in x[::97]:
            assert REF.float_to_bf16(v) == int(lit.float_to_bf16(v))


def test_gemm_bf16_closed_forms_fast_and_ref():
    from composable_kernel_amd.host_tensor import uniform_bf16
    # ones: every entry is K, exact in bf16 up to 256
    a = np.full((5, 192), 0x3F80, np.uint16)
    b = np.asfortranarray(np.full((192, 7), 0x3F80, np.uint16))
    np.testing.assert_array_equal(lit.gemm_bf16(a, b), np.full((5, 7), lit.float_to_bf16(np.float32(192.0)), np.uint16))
    # K = 257 ones -> 257 is not a bf16 (8 significant bits): tie between 256 and 258 -> 256
    a = np.full((2, 257), 0x3F80, np.uint16)
    b = np.asfortranarray(np.full((257, 3), 0x3F80, np.uint16))
    assert np.all(fast.bf16_to_f32(lit.gemm_bf16(a, b)) == 256.0)
    a = uniform_bf16((33, 160), -1, 1, 21)
    b = np.asfortranarray(uniform_bf16((160, 29), -1, 1, 22))
    c = lit.gemm_bf16(a, b)
    exact = fast.bf16_to_f32(a).astype(np.float64) @ fast.bf16_to_f32(b).astype(np.float64)
    assert np.all(np.abs(fast.bf16_to_f32(c) - exact) <= 2.0 ** -8 * np.abs(exact) + 1e-4)
    f = fast.bf16_to_f32(fast.gemm_bf16(a, b))
    assert np.all(np.abs(fast.bf16_to_f32(c) - f) <= 1e-2 + 1e-2 * np.abs(f))
    if REF is not None:
        np.testing.assert_array_equal(REF.gemm_bf16(a, b), c)


def test_gemm_softmax_gemm_closed_forms():
    """What the mathematics fixes: zero scores give the uniform distribution; under the upper-triangle mask
    row 0 sees only column 0; a dominant score selects its row of B1; the scale multiplies the scores."""
    G, M, N, K, O = 2, 24, 32, 16, 8
    b1 = (np.arange(G * N * O).reshape(G, N, O) % 7).astype(np.float16)
    a0 = np.zeros((G, M, K), np.float16)
    b0 = uniform_f16((G, K, N), -1, 1, 71)
    # uniform: p = half(1/32) = 2^-5 exactly, C = mean over n of B1 (small integers / 32: exact in fp16)
    np.testing.assert_array_equal(lit.batched_gemm_softmax_gemm_f16(a0, b0, b1),
                                  np.broadcast_to(b1.astype(np.float32).mean(axis=1, keepdims=True), (G, M, O)).astype(np.float16))
    # mask: row m averages rows 0..m of B1; row 0 is B1[0] exactly, row 3 the mean of four rows
    c = lit.batched_gemm_softmax_gemm_f16(a0, b0, b1, mask_upper=True)
    np.testing.assert_array_equal(c[:, 0], b1[:, 0])
    np.testing.assert_array_equal(c[:, 3], b1[:, :4].astype(np.float32).mean(axis=1).astype(np.float16))
    # dominant score: A = e_k rows, B0 = 40 * identity-like -> softmax is one-hot to within exp(-40)
    a = np.zeros((G, M, K), np.float16)
    a[:, np.arange(M), np.arange(M) % K] = 1
    b0h = np.zeros((G, K, N), np.float16)
    b0h[:, np.arange(K), (np.arange(K) * 2) % N] = 40
    c = lit.batched_gemm_softmax_gemm_f16(a, b0h, b1)
    np.testing.assert_array_equal(c, b1[:, ((np.arange(M) % K) * 2) % N])
    # the scale acts on the scores: scale 0 is the uniform case whatever A and B0 hold
    an = uniform_f16((G, M, K), -1, 1, 72)
    np.testing.assert_array_equal(lit.batched_gemm_softmax_gemm_f16(an, b0, b1, scale=0.0),
                                  lit.batched_gemm_softmax_gemm_f16(a0, b0, b1))


@pytest.mark.parametrize("mask", [False, True])
def test_gemm_softmax_gemm_against_scipy_fast_and_ref(mask):
    """float64 softmax (scipy) with an fp16 rounding of the probabilities, the numpy form, and -- bit for bit --
    the reference's own ReferenceBatchedGemm / Scale / ReferenceSoftmax chain where it is built."""
    from scipy.special import softmax
    for (G, M, N, K, O), scale in [((3, 40, 72, 24, 16), 0.125), ((2, 65, 33, 64, 40), 1.0), ((1, 7, 130, 8, 8), 0.5)]:
        a = uniform_f16((G, M, K), -1, 1, 80 + M)
        b0 = uniform_f16((G, N, K), -1, 1, 81 + N).transpose(0, 2, 1)      # stored [G,N,K]
        b1 = uniform_f16((G, N, O), -1, 1, 82 + O)
        c = lit.batched_gemm_softmax_gemm_f16(a, b0, b1, scale, mask)
        x = scale * np.matmul(a.astype(np.float64), b0.astype(np.float64))
        if mask:
            x = np.where(np.arange(N)[None, None, :] > np.arange(M)[None, :, None], -np.inf, x)
        p = softmax(x, axis=2).astype(np.float16)
        want = np.matmul(p.astype(np.float64), b1.astype(np.float64))
        assert np.abs(c.astype(np.float64) - want).max() < 2e-3
        bad, max_err = lit.check_err_f16(fast.batched_gemm_softmax_gemm_f16(a, b0, b1, scale, mask), c, 1e-2, 1e-2)
        assert bad == 0, max_err
        if REF is not None:
            np.testing.assert_array_equal(REF.batched_gemm_softmax_gemm_f16(a, b0, b1, scale, mask).view(np.uint16),
                                          c.view(np.uint16))
        # thread count is unobservable
        np.testing.assert_array_equal(lit.batched_gemm_softmax_gemm_f16(a, b0, b1, scale, mask, nthreads=1), c)
