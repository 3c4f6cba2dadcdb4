"""The 256 x 256 tile instance has two kernel bodies for dense K-contiguous GEMMs with a plain epilogue: eight waves
(two per SIMD, 128 x 64 wave tiles) and four waves (one per SIMD, 128 x 128 wave tiles, accumulators in AccVGPRs).
ckx_set_big_tile_waves forces either; the library chooses by problem size otherwise. Here the four-wave body runs every
kind of shape -- ragged M and N, K tails, K of one tile and less, more tiles than CUs, padded C rows -- through the C ABI
against the CPU oracle (int8 bit-exact in all three epilogues, fp16 / bf16 at rtol = atol = 1e-2 and bit-exact on integer
operands), and against the eight-wave body bit for bit: both add the K tiles in the same order.
"""
import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_bf16, uniform_f16, uniform_int8
from oracle import fast, lit

pytestmark = pytest.mark.gpu


@pytest.fixture
def waves():
    def _set(n):
        capi.lib().ckx_set_big_tile_waves(int(n))
    yield _set
    capi.lib().ckx_set_big_tile_waves(0)


def _gemm_bf16(a, b_nk, instance=0):
    import torch
    import gpu_util
    M, K = a.shape
    N = b_nk.shape[0]
    da, db = torch.from_numpy(a.view(np.int16)).cuda(), torch.from_numpy(b_nk.view(np.int16)).cuda()
    dc = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
    op = ck.DeviceGemmBF16(instance)
    arg = op.MakeArgumentPointer(da, db, dc, M, N, K, K, K, N)
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    return dc.cpu().numpy().view(np.uint16)


SHAPES = [(256, 256, 128), (256, 256, 64), (512, 768, 1024), (300, 520, 208), (1, 16, 16), (255, 257, 4096),
          (513, 80, 1040), (1024, 1024, 2064), (77, 1000, 144)]
OPS = {"pass": (ck.PassThrough(), lit.EPI_PASSTHROUGH, 1.0, 1.0),
       "ck": (ck.RequantReluRequant(0.02, 0.4), lit.EPI_REQUANT_CK, 0.02, 0.4),
       "rnd": (ck.RequantReluRequant(0.5, 0.03, rounded=True), lit.EPI_REQUANT_RND, 0.5, 0.03)}


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("op", list(OPS))
def test_int8_four_wave_body_bit_exact(waves, shape, op):
    import gpu_util
    M, N, K = shape
    a = uniform_int8((M, K), -5, 5, 3100 + M)
    b_nk = uniform_int8((N, K), -5, 5, 3101 + N)
    c_op, epi, sg, sr = OPS[op]
    waves(4)
    out = gpu_util.gemm_i8(a, b_nk, c_op, 0, ldc=N + 16)
    np.testing.assert_array_equal(out, fast.gemm_i8(a, b_nk.T, epi, sg, sr))
    waves(8)
    np.testing.assert_array_equal(gpu_util.gemm_i8(a, b_nk, c_op, 0, ldc=N + 16), out)


@pytest.mark.parametrize("shape", SHAPES)
def test_fp16_four_wave_body(waves, shape):
    import gpu_util
    M, N, K = shape
    a = uniform_f16((M, K), -1, 1, 3200 + M)
    b_nk = uniform_f16((N, K), -1, 1, 3201 + N)
    waves(4)
    out = gpu_util.gemm_f16(a, b_nk, 0)
    bad, max_err = lit.check_err_f16(out, fast.gemm_f16(a, b_nk.T), 1e-2, 1e-2)
    assert bad == 0, max_err
    waves(8)
    np.testing.assert_array_equal(gpu_util.gemm_f16(a, b_nk, 0).view(np.uint16), out.view(np.uint16))
    # integer operands: every partial sum is exact, the result is the integer matrix product
    ai = uniform_int8((M, K), -3, 3, 3202).astype(np.float16)
    bi = uniform_int8((N, K), -3, 3, 3203).astype(np.float16)
    waves(4)
    want = (ai.astype(np.float32) @ bi.T.astype(np.float32)).astype(np.float16)
    np.testing.assert_array_equal(gpu_util.gemm_f16(ai, bi, 0), want)


@pytest.mark.parametrize("shape", [(256, 256, 128), (300, 520, 208), (513, 80, 1040), (255, 257, 4096)])
def test_bf16_four_wave_body(waves, shape):
    M, N, K = shape
    a = uniform_bf16((M, K), -1, 1, 3300 + M)
    b_nk = uniform_bf16((N, K), -1, 1, 3301 + N)
    waves(4)
    out = _gemm_bf16(a, b_nk)
    o, r = fast.bf16_to_f32(out), fast.bf16_to_f32(lit.gemm_bf16(a, b_nk.T) if M * N * K < 3e7 else fast.gemm_bf16(a, b_nk.T))
    assert np.all(np.isfinite(o)) and np.all(np.abs(o - r) <= 1e-2 + 1e-2 * np.abs(r))
    waves(8)
    np.testing.assert_array_equal(_gemm_bf16(a, b_nk), out)


def test_more_tiles_than_cus_and_empty_k(waves):
    """17 x 17 tiles of 256 x 256 (289 workgroups' worth on 256 CUs: some workgroups take a second tile, with the C
    stores of the first still in flight), and K = 0 (C = epilogue(0))."""
    import gpu_util
    M = N = 4352
    K = 256
    a = uniform_int8((M, K), -5, 5, 3400)
    b_nk = uniform_int8((N, K), -5, 5, 3401)
    c_op, epi, sg, sr = OPS["rnd"]
    waves(4)
    np.testing.assert_array_equal(gpu_util.gemm_i8(a, b_nk, c_op, 0), fast.gemm_i8(a, b_nk.T, epi, sg, sr))
    af = uniform_f16((M, 192), -1, 1, 3402)
    bf = uniform_f16((N, 192), -1, 1, 3403)
    bad, max_err = lit.check_err_f16(gpu_util.gemm_f16(af, bf, 0), fast.gemm_f16(af, bf.T), 1e-2, 1e-2)
    assert bad == 0, max_err
    import torch
    d = torch.ones(1 << 12, dtype=torch.float16, device="cuda")          # never read: K = 0
    c = torch.full((300, 260), float("nan"), dtype=torch.float16, device="cuda")
    op = ck.DeviceGemmF16(0)
    arg = op.MakeArgumentPointer(d, d, c, 300, 260, 0, 8, 8, 260)
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    assert not c.cpu().numpy().any()


def test_automatic_choice_is_either_body_with_identical_results(waves):
    """Whichever body the library picks (by data type and K length), the results do not depend on it."""
    import gpu_util
    for K in (128, 2048):
        a = uniform_f16((512, K), -1, 1, 3500 + K)
        b_nk = uniform_f16((512, K), -1, 1, 3501 + K)
        waves(0)
        auto = gpu_util.gemm_f16(a, b_nk, 0)
        for w in (4, 8):
            waves(w)
            np.testing.assert_array_equal(gpu_util.gemm_f16(a, b_nk, 0).view(np.uint16), auto.view(np.uint16))
    assert capi.lib().ckx_set_big_tile_waves(0) == 8
    assert capi.lib().ckx_set_big_tile_waves(5) == 0 and capi.lib().ckx_set_big_tile_waves(0) == 0   # 5 is not a choice


@pytest.mark.parametrize("shape", [(256, 256, 128), (300, 520, 208), (1024, 1024, 1040), (77, 1000, 144)])
def test_fp16_d_operand_epilogues_on_both_bodies(waves, shape):
    """AddRelu (C rounded first) and Bilinear run on either body, bit-identical; the functors with two D tensors
    (AddReluAdd, AddAddFastGelu) stay on the eight-wave body whatever the knob says. All against the oracle; bias row
    and full D tensors, padded strides."""
    import torch
    import gpu_util
    M, N, K = shape
    a = uniform_f16((M, K), -0.5, 0.5, 3600 + M)
    b_nk = uniform_f16((N, K), -0.5, 0.5, 3601 + N)
    row = uniform_f16((1, N), -2, 2, 3602)
    full = uniform_f16((M, N + 8), -2, 2, 3603)
    full2 = uniform_f16((M, N), -2, 2, 3604)
    acc = a.astype(np.float32) @ b_nk.T.astype(np.float32)
    cases = [
        (ck.AddRelu(), [row], [0], fast.gemm_f16_add_relu(a, b_nk.T, row)),
        (ck.AddRelu(), [full], [N + 8], fast.gemm_f16_add_relu(a, b_nk.T, full[:, :N])),
        (ck.AddReluAdd(), [row, full], [0, N + 8],
         (np.maximum(acc + row.astype(np.float32), 0) + full[:, :N].astype(np.float32)).astype(np.float16)),
        (ck.AddReluAdd(), [full2, full], [N, N + 8],
         (np.maximum(acc + full2.astype(np.float32), 0) + full[:, :N].astype(np.float32)).astype(np.float16)),
        (ck.Bilinear(0.75, -1.5), [full], [N + 8], fast.gemm_f16_bilinear(a, b_nk.T, full[:, :N], 0.75, -1.5)),
        (ck.Bilinear(2.0, 0.5), [row], [0], fast.gemm_f16_bilinear(a, b_nk.T, row, 2.0, 0.5)),
        (ck.AddAddFastGelu(), [row, full], [0, N + 8], fast.gemm_f16_add_add_fastgelu(a, b_nk.T, row, full[:, :N])),
        (ck.AddAddFastGelu(), [full, full2], [N + 8, N], fast.gemm_f16_add_add_fastgelu(a, b_nk.T, full[:, :N], full2)),
    ]
    da, db = gpu_util.dev(a), gpu_util.dev(b_nk)
    for functor, ds, strides, want in cases:
        outs = []
        for w in (4, 8):
            waves(w)
            dds = [gpu_util.dev(d) for d in ds]
            de = torch.full((M, N + 24), 77.0, dtype=torch.float16, device="cuda")
            op = ck.DeviceGemmMultipleDF16(0)
            arg = op.MakeArgumentPointer(da, db, dds, de, M, N, K, K, K, strides, N + 24, None, None, functor)
            assert op.IsSupportedArgument(arg), capi.last_error()
            op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
            torch.cuda.synchronize()
            out = de.cpu().numpy()
            assert np.all(out[:, N:] == 77.0)
            outs.append(out[:, :N].copy())
        bad, max_err = lit.check_err_f16(outs[0], want, 1e-2, 1e-2)
        assert bad == 0, (type(functor).__name__, max_err)
        np.testing.assert_array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))


@pytest.mark.parametrize("case", [(3, 256, 256, 128, (0, 0, 0), False), (3, 130, 200, 272, (16, 32, 8), False),
                                  (5, 300, 72, 1040, (0, 0, 24), True), (20, 512, 256, 1024, (0, 0, 0), False)])
def test_strided_batches_on_both_bodies(waves, case):
    """DeviceBatchedGemm on tile instance 0: the tiles of all batches are one work list for either body (padded batch
    strides, a B matrix shared by all batches, more tiles than CUs in the last case)."""
    import torch
    from test_batched_gemm_gpu import _run as run_batched
    G, M, N, K, bs, share_b = case
    a = uniform_int8((G, M, K), -8, 8, 3700 + M)
    b = uniform_int8((G, N, K), -8, 8, 3701 + N)
    if share_b:
        b[:] = b[0]
    c_op = ck.RequantReluRequant(0.02, 0.4, rounded=True)
    af, bf = uniform_f16((G, M, K), -1, 1, 3702), uniform_f16((G, N, K), -1, 1, 3703)
    if share_b:
        bf[:] = bf[0]
    outs = {}
    for w in (4, 8):
        waves(w)
        outs[w] = (run_batched(ck.DeviceBatchedGemmInt8(0), a, b, torch.int8, bs, share_b, c_op),
                   run_batched(ck.DeviceBatchedGemmF16(0), af, bf, torch.float16, bs, share_b))
    for g in range(G):
        np.testing.assert_array_equal(outs[4][0][g], fast.gemm_i8(a[g], b[g].T, lit.EPI_REQUANT_RND, 0.02, 0.4))
        bad, max_err = lit.check_err_f16(outs[4][1][g], fast.gemm_f16(af[g], bf[g].T), 1e-2, 1e-2)
        assert bad == 0, max_err
    np.testing.assert_array_equal(outs[4][0], outs[8][0])
    np.testing.assert_array_equal(outs[4][1].view(np.uint16), outs[8][1].view(np.uint16))


def test_padded_operand_strides_on_both_bodies(waves):
    """Leading dimensions larger than K (multiples of 16 bytes) and a padded C: the rows the kernels fetch are the
    problem's, whatever lies between them."""
    import torch
    import gpu_util
    M, N, K = 520, 300, 328
    lda, ldb, ldc = K + 8, K + 24, N + 8
    a = np.full((M, lda), np.float16(7.0))
    b = np.full((N, ldb), np.float16(-9.0))
    a[:, :K] = uniform_f16((M, K), -1, 1, 3800)
    b[:, :K] = uniform_f16((N, K), -1, 1, 3801)
    want = fast.gemm_f16(a[:, :K], b[:, :K].T)
    outs = []
    for w in (4, 8):
        waves(w)
        da, db = gpu_util.dev(a), gpu_util.dev(b)
        dc = torch.full((M, ldc), 77.0, dtype=torch.float16, device="cuda")
        op = ck.DeviceGemmF16(0)
        arg = op.MakeArgumentPointer(da, db, dc, M, N, K, lda, ldb, ldc)
        assert op.IsSupportedArgument(arg), capi.last_error()
        op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
        torch.cuda.synchronize()
        out = dc.cpu().numpy()
        assert np.all(out[:, N:] == 77.0)
        outs.append(out[:, :N].copy())
    bad, max_err = lit.check_err_f16(outs[0], want, 1e-2, 1e-2)
    assert bad == 0, max_err
    np.testing.assert_array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))


@pytest.mark.parametrize("seed", range(24))
def test_seeded_random_problems_on_the_four_wave_body(waves, seed):
    """Random extents, K tails of every 16-byte multiple, padded leading dimensions and C rows, forced onto the four-wave
    body: int8 (rounded requant) bit-exact against the oracle, fp16 on small integers bit-exact
    against the exact product (every partial sum is an integer below 2^24)."""
    import torch
    import gpu_util
    rng = np.random.default_rng(4100 + seed)
    M, N = int(rng.integers(1, 1100)), int(rng.integers(1, 1100))
    if seed % 6 == 0:
        M = int(rng.integers(2200, 4200))            # more tiles than the workgroups of a launch now and then
    waves(4)
    if seed % 2 == 0:
        K = 16 * int(rng.integers(1, 160))
        lda, ldb, ldc = K + 16 * int(rng.integers(0, 3)), K + 16 * int(rng.integers(0, 3)), N + int(rng.integers(0, 20))
        a = rng.integers(-15, 16, (M, lda), dtype=np.int8)
        b = rng.integers(-15, 16, (N, ldb), dtype=np.int8)
        sg, sr = 0.02, 0.75
        da, db = gpu_util.dev(a), gpu_util.dev(b)
        dc = torch.full((M, ldc), 77, dtype=torch.int8, device="cuda")
        op = ck.DeviceGemmInt8(0)
        arg = op.MakeArgumentPointer(da, db, dc, M, N, K, lda, ldb, ldc, ck.PassThrough(), ck.PassThrough(),
                                     ck.RequantReluRequant(sg, sr, rounded=True))
        want = fast.gemm_i8(a[:, :K], b[:, :K].T, lit.EPI_REQUANT_RND, sg, sr)
    else:
        K = 8 * int(rng.integers(1, 200))
        lda, ldb, ldc = K + 8 * int(rng.integers(0, 3)), K + 8 * int(rng.integers(0, 3)), N + int(rng.integers(0, 20))
        a = rng.integers(-4, 5, (M, lda)).astype(np.float16)
        b = rng.integers(-4, 5, (N, ldb)).astype(np.float16)
        da, db = gpu_util.dev(a), gpu_util.dev(b)
        dc = torch.full((M, ldc), 77.0, dtype=torch.float16, device="cuda")
        op = ck.DeviceGemmF16(0)
        arg = op.MakeArgumentPointer(da, db, dc, M, N, K, lda, ldb, ldc)
        want = (a[:, :K].astype(np.int64) @ b[:, :K].astype(np.int64).T).astype(np.float32).astype(np.float16)
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    out = dc.cpu().numpy()
    assert np.all(out[:, N:] == 77), "wrote outside the C rows"
    np.testing.assert_array_equal(out[:, :N], want)
