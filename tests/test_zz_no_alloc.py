"""GPU parity of ckx_gemm_i8_splitk_noalloc: the int8 split-K GEMM whose workspace is the library's
own static device array (for callers that cannot allocate). It is checked, through the C ABI, against
ckx_gemm_i8_splitk with a workspace of the caller's on the same inputs -- bit-exact, as for all int8
work -- on two calls in a row, the second on a smaller problem (the static array then still holds the
first call's slices), and against the CPU form of the reference GEMM."""
import ctypes as C

import numpy as np
import pytest

from composable_kernel_amd import capi
from composable_kernel_amd.host_tensor import uniform_int8
from oracle import fast, lit

pytestmark = pytest.mark.gpu

SG, SR = 0.02, 0.4


def _both(M, N, K, k_batch, seed, instance=capi.INSTANCE_AUTO):
    """(output of the allocation-free entry point, output of ckx_gemm_i8_splitk, expected)"""
    import torch
    import gpu_util
    L = capi.lib()
    a = uniform_int8((M, K), -8, 8, seed)
    b_nk = uniform_int8((N, K), -8, 8, seed + 1)
    da, db = gpu_util.dev(a), gpu_util.dev(b_nk)
    need = int(L.ckx_gemm_splitk_workspace_bytes(capi.OP_GEMM_I8, M, N, K, k_batch))
    assert 0 < need <= capi.STATIC_WORKSPACE_BYTES
    ws = torch.full((need,), 0x55, dtype=torch.uint8, device="cuda")
    c_ref = torch.full((M, N), 77, dtype=torch.int8, device="cuda")
    c_new = torch.full((M, N), 78, dtype=torch.int8, device="cuda")
    s = C.c_void_p(gpu_util.stream())
    shape = (M, N, K, K, K, N, capi.ROW_MAJOR, capi.COL_MAJOR, capi.ROW_MAJOR, capi.EPI_REQUANT_RND, SG, SR, instance, k_batch)
    capi.check(L.ckx_gemm_i8_splitk(da.data_ptr(), db.data_ptr(), c_ref.data_ptr(), *shape, ws.data_ptr(), need, s))
    capi.check(L.ckx_gemm_i8_splitk_noalloc(da.data_ptr(), db.data_ptr(), c_new.data_ptr(), *shape, s))
    torch.cuda.synchronize()
    return c_new.cpu().numpy(), c_ref.cpu().numpy(), fast.gemm_i8(a, b_nk.T, lit.EPI_REQUANT_RND, SG, SR)


def test_noalloc_split_k_matches_the_workspace_entry_point_twice_in_a_row():
    # 4 runs of 8 K tiles, slices of 4 x 200 x 328 x 4 bytes; then a smaller problem, 3 runs
    for (M, N, K, kb, seed) in [(200, 328, 4096, 4, 300), (72, 136, 1536, 3, 310)]:
        got, ref, want = _both(M, N, K, kb, seed)
        np.testing.assert_array_equal(got, ref)
        np.testing.assert_array_equal(got, want)


def test_noalloc_entry_point_allocates_no_device_memory():
    """hipMemGetInfo before and after two calls (the first resolves the static array's address): the free figure
    does not move. Operands and the output are allocated beforehand."""
    import torch
    import gpu_util
    L = capi.lib()
    M, N, K, kb = 136, 200, 2048, 4
    da = gpu_util.dev(uniform_int8((M, K), -8, 8, 330))
    db = gpu_util.dev(uniform_int8((N, K), -8, 8, 331))
    dc = torch.zeros((M, N), dtype=torch.int8, device="cuda")
    s = C.c_void_p(gpu_util.stream())
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(2):
        capi.check(L.ckx_gemm_i8_splitk_noalloc(da.data_ptr(), db.data_ptr(), dc.data_ptr(), M, N, K, K, K, N, capi.ROW_MAJOR,
                                                capi.COL_MAJOR, capi.ROW_MAJOR, capi.EPI_REQUANT_RND, SG, SR, capi.INSTANCE_AUTO,
                                                kb, s))
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0


def test_noalloc_argument_errors_are_answered_like_the_workspace_entry_point():
    """Bad arguments and empty problems come back before any device work: the codes of ckx_gemm_i8_splitk."""
    L = capi.lib()
    s = C.c_void_p(0)
    call = lambda M, N, K, bl, kb: L.ckx_gemm_i8_splitk_noalloc(0, 0, 0, M, N, K, K, K, N, capi.ROW_MAJOR, bl, capi.ROW_MAJOR,
                                                            capi.EPI_REQUANT_RND, SG, SR, capi.INSTANCE_AUTO, kb, s)
    assert call(64, 64, 1024, capi.COL_MAJOR, 9) == capi.UNSUPPORTED
    assert call(64, 64, 1024, 7, 2) == capi.INVALID_VALUE
    assert call(0, 64, 1024, capi.COL_MAJOR, 2) == capi.OK
    assert call(64, 64, 1024, capi.COL_MAJOR, 0) == capi.INVALID_VALUE


def test_noalloc_split_k_at_the_size_limit_and_beyond():
    import torch
    import gpu_util
    L = capi.lib()
    # 8 runs x 1024 x 1024 x 4 bytes = exactly the 32 MiB of the static array
    got, ref, want = _both(1024, 1024, 1024, 8, 320, instance=0)
    np.testing.assert_array_equal(got, ref)
    np.testing.assert_array_equal(got, want)
    # one row more does not fit: refused with a message, nothing launched, C untouched
    M, N, K = 1025, 1024, 1024
    da = torch.zeros((M, K), dtype=torch.int8, device="cuda")
    db = torch.zeros((N, K), dtype=torch.int8, device="cuda")
    dc = torch.full((M, N), 79, dtype=torch.int8, device="cuda")
    st = L.ckx_gemm_i8_splitk_noalloc(da.data_ptr(), db.data_ptr(), dc.data_ptr(), M, N, K, K, K, N, capi.ROW_MAJOR,
                                      capi.COL_MAJOR, capi.ROW_MAJOR, capi.EPI_REQUANT_RND, SG, SR, 0, 8,
                                      C.c_void_p(gpu_util.stream()))
    assert st == capi.UNSUPPORTED and "static workspace" in capi.last_error()
    torch.cuda.synchronize()
    assert bool((dc == 79).all())
