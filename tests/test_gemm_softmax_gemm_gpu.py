"""GPU parity: batched fused GEMM + softmax + GEMM ("attention", fp16) through the C ABI against the CPU
oracle -- ReferenceBatchedGemm with element_wise::Scale, the upper-triangle mask, ReferenceSoftmax over n
(reference_softmax.hpp:56-117) and a second ReferenceBatchedGemm, the chain upstream's
batched_gemm_scale_softmax_gemm example verifies with. The fused operator is absent from the reference
snapshot; the oracle chain is pinned bit for bit against those reference pieces in tests/test_oracle.py.
This row is TOLERANCE-ONLY, by construction: rtol = atol = 1e-2. The kernel rounds the unnormalised
probabilities exp(s - max) to fp16 (they are the A operand of the second MFMA GEMM) and divides the fp32
result by the row sum afterwards; the reference divides first and rounds the normalised probabilities. The two
round different numbers, so outputs differ by a few fp16 units in the last place of the probabilities (relative
2^-11 each, accumulated over n): a comparison at 1e-3 fails on a share of the elements for this reason alone,
and no reordering inside the kernel can make the row bit-exact without giving up the fused second GEMM.
What the mathematics fixes exactly is still checked exactly (uniform rows, one-hot rows, the masked first row)."""
import numpy as np
import pytest

import composable_kernel_amd as ck
from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_f16
from oracle import fast, lit

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def _close(out, ref):
    assert np.all(np.isfinite(out.astype(np.float32)))
    bad, max_err = lit.check_err_f16(out, ref, RTOL, ATOL)
    assert bad == 0, f"{bad} outside tolerance, max err {max_err}"


def _run(a_gmk, b0_gnk, b1_gno, scale=1.0, mask=False, instance=capi.INSTANCE_AUTO, pad=(0, 0, 0, 0)):
    """pad: extra elements per row of A, B0, B1, C (row strides larger than the extents)."""
    import torch
    import gpu_util
    G, M, K = a_gmk.shape
    N, O = b0_gnk.shape[1], b1_gno.shape[2]

    def padded(x, p):
        out = np.zeros(x.shape[:2] + (x.shape[2] + p,), np.float16)
        out[..., :x.shape[2]] = x
        return out

    ha, hb0, hb1 = padded(a_gmk, pad[0]), padded(b0_gnk, pad[1]), padded(b1_gno, pad[2])
    da, db0, db1 = (torch.from_numpy(x.view(np.int16)).cuda() for x in (ha, hb0, hb1))
    dc = torch.full((G, M, O + pad[3]), 0x7E00, dtype=torch.int16, device="cuda")
    op = ck.DeviceBatchedGemmSoftmaxGemmF16(instance, MaskOutUpperTriangle=mask)
    arg = op.MakeArgumentPointer(da, db0, db1, dc, M, N, K, O, G, K + pad[0], K + pad[1], O + pad[2], O + pad[3],
                                 M * (K + pad[0]), N * (K + pad[1]), N * (O + pad[2]), M * (O + pad[3]),
                                 None, None, ck.Scale(scale))
    assert op.IsSupportedArgument(arg), capi.last_error()
    op.MakeInvokerPointer().Run(arg, ck.StreamConfig(gpu_util.stream()))
    torch.cuda.synchronize()
    out = dc.cpu().numpy().view(np.float16)
    if pad[3]:
        assert np.all(out[..., O:].view(np.uint16) == 0x7E00), "wrote outside the C rows"
    return out[..., :O]


SHAPES = [
    # G, M, N, K, O
    (3, 128, 128, 64, 64), (2, 200, 136, 64, 64), (2, 96, 512, 32, 64), (1, 130, 260, 128, 128),
    (2, 64, 72, 40, 24), (5, 16, 8, 8, 8), (1, 256, 300, 96, 128), (2, 40, 1, 16, 16), (1, 1, 257, 64, 64),
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("instance", [capi.INSTANCE_AUTO, 1, 2])
def test_gemm_softmax_gemm_shapes(shape, mask, instance):
    G, M, N, K, O = shape
    a = uniform_f16((G, M, K), -1, 1, 1900 + M)
    b0_gnk = uniform_f16((G, N, K), -1, 1, 1901 + N)
    b1 = uniform_f16((G, N, O), -1, 1, 1902 + O)
    scale = 1.0 / np.sqrt(K)
    out = _run(a, b0_gnk, b1, scale, mask, instance)
    _close(out, lit.batched_gemm_softmax_gemm_f16(a, b0_gnk.transpose(0, 2, 1), b1, scale, mask))


def test_gemm_softmax_gemm_closed_forms():
    """Zero scores: the uniform distribution, C = mean of B1's rows (exact: small integers over a power of
    two). Upper-triangle mask: row m averages rows 0..m, row 0 is B1[0] exactly. A dominant score selects
    one row of B1 exactly."""
    G, M, N, K, O = 2, 160, 256, 32, 64
    b1 = (np.arange(G * N * O).reshape(G, N, O) % 7).astype(np.float16)
    a0 = np.zeros((G, M, K), np.float16)
    b0 = uniform_f16((G, N, K), -1, 1, 71)
    out = _run(a0, b0, b1)
    np.testing.assert_array_equal(out, np.broadcast_to(b1.astype(np.float32).mean(axis=1, keepdims=True),
                                                       (G, M, O)).astype(np.float16))
    out = _run(a0, b0, b1, mask=True)
    np.testing.assert_array_equal(out[:, 0], b1[:, 0])
    for m in (1, 3, 7, 127, 159):        # m + 1 a power of two, or within fp16 rounding otherwise
        want = b1[:, :m + 1].astype(np.float64).mean(axis=1)
        assert np.abs(out[:, m].astype(np.float64) - want).max() <= 4e-3
    a = np.zeros((G, M, K), np.float16)
    a[:, np.arange(M), np.arange(M) % K] = 1
    b0h = np.zeros((G, N, K), np.float16)
    b0h[:, (np.arange(K) * 5) % N, np.arange(K)] = 40
    out = _run(a, b0h, b1)
    np.testing.assert_array_equal(out, b1[:, ((np.arange(M) % K) * 5) % N])


def test_gemm_softmax_gemm_running_maximum_is_rescaled():
    """The row maximum sits in the LAST 128-column step and the early steps hold large negative scores, and
    the other way round: the one-pass softmax must rescale what it accumulated."""
    G, M, N, K, O = 1, 64, 512, 16, 32
    a = np.zeros((G, M, K), np.float16)
    a[..., 0] = 1
    b1 = uniform_f16((G, N, O), -1, 1, 5)
    for ramp in (np.linspace(-30, 8, N), np.linspace(8, -30, N)):
        b0 = np.zeros((G, N, K), np.float16)
        b0[0, :, 0] = ramp.astype(np.float16)
        out = _run(a, b0, b1)
        _close(out, lit.batched_gemm_softmax_gemm_f16(a, b0.transpose(0, 2, 1), b1))
        # scores far apart (neighbours differ by 0.074 * 300): the result is the row of B1 at the maximum
        out = _run(a, b0, b1, scale=300.0)
        np.testing.assert_array_equal(out[0], np.broadcast_to(b1[0, int(np.argmax(b0[0, :, 0]))], (M, O)))


def test_gemm_softmax_gemm_negative_scale():
    """A negative scale turns the softmax towards the SMALLEST raw score (the kernel moves the sign into A)."""
    G, M, N, K, O = 2, 96, 300, 32, 32
    a = uniform_f16((G, M, K), -1, 1, 21)
    b0_gnk = uniform_f16((G, N, K), -1, 1, 22)
    b1 = uniform_f16((G, N, O), -1, 1, 23)
    for mask in (False, True):
        out = _run(a, b0_gnk, b1, -0.7, mask)
        _close(out, lit.batched_gemm_softmax_gemm_f16(a, b0_gnk.transpose(0, 2, 1), b1, -0.7, mask))
        # same as a positive scale on the negated A
        np.testing.assert_array_equal(out.view(np.uint16), _run(-a, b0_gnk, b1, 0.7, mask).view(np.uint16))


def test_gemm_softmax_gemm_padded_strides_and_scale_zero():
    G, M, N, K, O = 3, 72, 200, 64, 48
    a = uniform_f16((G, M, K), -1, 1, 11)
    b0_gnk = uniform_f16((G, N, K), -1, 1, 12)
    b1 = uniform_f16((G, N, O), -1, 1, 13)
    out = _run(a, b0_gnk, b1, 0.125, False, pad=(8, 16, 24, 8))
    _close(out, lit.batched_gemm_softmax_gemm_f16(a, b0_gnk.transpose(0, 2, 1), b1, 0.125))
    # scale 0 makes the scores irrelevant: same result as A = 0
    np.testing.assert_array_equal(_run(a, b0_gnk, b1, 0.0).view(np.uint16),
                                  _run(np.zeros_like(a), b0_gnk, b1).view(np.uint16))


@pytest.mark.parametrize("mask", [False, True])
def test_gemm_softmax_gemm_config5_shape(mask):
    """Benchmark configuration 5's shapes with the softmax in between: batch 64, 512 x 512 scores, K = O = 64."""
    G, M, N, K, O = 64, 512, 512, 64, 64
    a = uniform_f16((G, M, K), -1, 1, 1910)
    b0_gnk = uniform_f16((G, N, K), -1, 1, 1911)
    b1 = uniform_f16((G, N, O), -1, 1, 1912)
    out = _run(a, b0_gnk, b1, 0.125, mask)
    _close(out, fast.batched_gemm_softmax_gemm_f16(a, b0_gnk.transpose(0, 2, 1), b1, 0.125, mask))
    for g in (0, 63):
        _close(out[g:g + 1], lit.batched_gemm_softmax_gemm_f16(a[g:g + 1], b0_gnk[g:g + 1].transpose(0, 2, 1),
                                                               b1[g:g + 1], 0.125, mask))
    # rows of the output are convex combinations of B1's rows
    assert np.all(out.astype(np.float32).max(axis=1) <= b1.astype(np.float32).max(axis=1) + 1e-3)
    # batches are independent
    perm = np.random.default_rng(4).permutation(G)
    np.testing.assert_array_equal(_run(a[perm], b0_gnk[perm], b1[perm], 0.125, mask).view(np.uint16),
                                  out[perm].view(np.uint16))


def test_gemm_softmax_gemm_refused_arguments_and_empty_sum():
    import torch
    d = torch.zeros(1 << 16, dtype=torch.int16, device="cuda")
    op = ck.DeviceBatchedGemmSoftmaxGemmF16()
    # K above 128 is not built; a non-finite scale is invalid
    assert not op.IsSupportedArgument(op.MakeArgumentPointer(d, d, d, d, 64, 64, 256, 64, 1, 256, 256, 64, 64, 0, 0, 0, 0))
    assert not op.IsSupportedArgument(op.MakeArgumentPointer(d, d, d, d, 64, 64, 64, 64, 1, 64, 64, 64, 64, 0, 0, 0, 0,
                                                             None, None, ck.Scale(float("inf"))))
    with pytest.raises(TypeError):
        op.MakeArgumentPointer(d, d, d, d, 64, 64, 64, 64, 1, 64, 64, 64, 64, 0, 0, 0, 0, None, None, ck.AddRelu())
    assert capi.lib().ckx_num_instances(capi.OP_BATCHED_GEMM_SOFTMAX_GEMM) == 3
    assert b"SoftmaxGemm" in capi.lib().ckx_instance_name(capi.OP_BATCHED_GEMM_SOFTMAX_GEMM, 0)
    # N = 0: an empty sum, C = 0
    out = _run(np.ones((1, 16, 8), np.float16), np.zeros((1, 0, 8), np.float16), np.zeros((1, 0, 8), np.float16))
    np.testing.assert_array_equal(out, np.zeros((1, 16, 8), np.float16))
