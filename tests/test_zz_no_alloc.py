"""The entry point that allocates nothing (its split-K scratch is a static device array) against the existing bmm entry
points, through the C ABI: two calls in a row, the second with a smaller input, bit for bit.  Needs an MI355X."""
import ctypes

import numpy as np
import pytest
import torch

from util import rand_i32, rand_i64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import kernel
    kernel.lib.zk_clear_error()
    vp, ll, ci = ctypes.c_void_p, ctypes.c_longlong, ctypes.c_int
    kernel.lib.int64_bmm_broadcast_noalloc.argtypes = [vp, vp, ci, vp, vp, ll, ll, ci, ci, ci, ci]
    return kernel


def _both(K, A, W, b_rs, c, want_r=True):
    """(C, R) of the existing entry point and of the one that allocates nothing, on the same device tensors"""
    Bd, M, Kd = A.shape
    N = W.shape[0]
    dA, dW = torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda()
    outs = []
    for noalloc in (False, True):
        C = torch.full((Bd, M, N), -7, dtype=torch.int64, device="cuda")
        R = torch.full((Bd, M, N), -7, dtype=torch.int64, device="cuda") if want_r else None
        rp = R.data_ptr() if want_r else None
        b32 = W.dtype == np.int32
        if noalloc:
            K.lib.int64_bmm_broadcast_noalloc(dA.data_ptr(), dW.data_ptr(), 1 if b32 else 0, C.data_ptr(), rp, b_rs, c, Bd, M, Kd, N)
        else:
            fn = K.lib.int64_32_bmm_broadcast_launcher if b32 else K.lib.int64_64_bmm_broadcast_launcher
            fn(dA.data_ptr(), dW.data_ptr(), C.data_ptr(), rp, 1, b_rs, c, Bd, M, Kd, N)
        K._check("bmm")
        outs.append((C, R))
    return outs


@pytest.mark.parametrize("w32", [False, True])
def test_no_alloc_entry_point_matches_the_existing_one(K, oracle, w32):
    rng = np.random.default_rng(300 + w32)
    mk = (lambda shape, bits: rand_i32(rng, shape, min(bits, 31))) if w32 else (lambda shape, bits: rand_i64(rng, shape, bits))
    # two calls in a row, the second smaller (fewer rows, columns, slices of K and batches): what the first call left in
    # the scratch must not show; then shapes without a K split, wide operands, a divisor on B, no remainder
    calls = [((2, 16, 7168), (576, 7168), 20, 16, 1, 29, True), ((1, 5, 1100), (130, 1100), 20, 16, 1, 29, True),
             ((1, 16, 64), (40, 64), 30, 30, 1, 0, True), ((1, 3, 2048), (3000, 2048), 63, 63, 1, 63, True),
             ((3, 9, 700), (33, 700), 37, 31, 256, 17, False), ((1, 16, 7168), (576, 7168), 28, 31, 1, 30, True)]
    pending = []
    for ashape, wshape, bits_a, bits_w, b_rs, c, want_r in calls:
        A, W = rand_i64(rng, ashape, bits_a), mk(wshape, bits_w)
        (C0, R0), (C1, R1) = _both(K, A, W, b_rs, c, want_r)
        pending.append((A, W, b_rs, c, C0, R0, C1, R1))
    for A, W, b_rs, c, C0, R0, C1, R1 in pending:          # (compared after all calls were queued: nothing waited in between)
        assert torch.equal(C0, C1), (A.shape, W.shape, "quotient")
        assert R0 is None or torch.equal(R0, R1), (A.shape, W.shape, "remainder")
        Ce, Re = oracle.int64_bmm_broadcast(A, W, 1, b_rs, c)
        assert np.array_equal(C1.cpu().numpy(), Ce) and (R1 is None or np.array_equal(R1.cpu().numpy(), Re))


def test_no_alloc_entry_point_allocates_nothing_and_rejects_what_it_cannot_take(K, oracle):
    rng = np.random.default_rng(310)
    A, W = rand_i64(rng, (1, 16, 7168), 20), rand_i64(rng, (576, 7168), 16)
    _both(K, A, W, 1, 29)                       # everything that is set up once has been set up
    dA, dW = torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda()
    C = torch.empty((1, 16, 576), dtype=torch.int64, device="cuda")
    R = torch.empty_like(C)
    torch.cuda.synchronize()
    held = K.workspace_bytes()
    free0 = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        K.lib.int64_bmm_broadcast_noalloc(dA.data_ptr(), dW.data_ptr(), 0, C.data_ptr(), R.data_ptr(), 1, 29, 1, 16, 7168, 576)
    torch.cuda.synchronize()
    K._check("noalloc")
    assert torch.cuda.mem_get_info()[0] == free0 and K.workspace_bytes() == held
    Ce, Re = oracle.int64_bmm_broadcast(A, W, 1, 1, 29)
    assert np.array_equal(C.cpu().numpy(), Ce) and np.array_equal(R.cpu().numpy(), Re)
    # beyond the limits: a clear error, nothing launched
    # (the last two: output counts whose product leaves 64 bits -- 2^30 * 16 * 2^30 wraps to 0 -- and one that wraps into the limit)
    for args in ((1, 29, 1, 17, 7168, 576), (1, 29, 1, 16, 64, (1 << 16) + 1), (3, 29, 1, 16, 7168, 576), (1, 64, 1, 16, 7168, 576),
                 (1, 29, 1 << 30, 16, 64, 1 << 30), (1, 29, (1 << 31) - 1, 16, 64, (1 << 31) - 1)):
        K.lib.int64_bmm_broadcast_noalloc(dA.data_ptr(), dW.data_ptr(), 0, C.data_ptr(), R.data_ptr(), *args)
        assert K.lib.zk_last_error() in (1, 3), args
        K.lib.zk_clear_error()
