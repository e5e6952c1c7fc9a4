"""Parity of the HIP library against the CPU oracle, bit for bit, through the C ABI (via the `kernel`
module, whose functions only allocate outputs and pass device pointers).  Needs an MI355X."""
import os

import numpy as np
import pytest
import torch

from util import rand_i32, rand_i64

pytestmark = pytest.mark.gpu

# ZK_TEST_SEEDS=n multiplies the seed ranges of the randomly drawn problem sets below (40, 20, 10 and 10 seeds by
# default), e.g. `ZK_TEST_SEEDS=200 python -m pytest tests/test_gpu_parity.py -m gpu -x -q -k seeded_random` runs 8000 +
# 4000 + 2000 + 2000 seeds and stops at the first mismatch
SEEDS = max(1, int(os.environ.get("ZK_TEST_SEEDS", "1") or 1))


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import kernel
    kernel.softmax_init_q19()
    kernel.softmax_init_q21()
    kernel.silu_init_q23()
    kernel.silu_init_q25()
    kernel.lib.zk_clear_error()
    yield kernel
    kernel.lib.zk_gemm_set_path(0)
    kernel.lib.zk_softmax_clobber_input(0)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.cpu().numpy()


PATHS = [pytest.param(1, id="valu"), pytest.param(2, id="mfma"), pytest.param(0, id="auto")]


# ------------------------------------------------------------------------------------ GEMM ------
def _gemm_case(K, oracle, path, A, W, a_rs, b_rs, c):
    K.lib.zk_gemm_set_path(path)
    C, R = K.int64_bmm_broadcast(dev(A), dev(W), a_rs, b_rs, c)
    Ce, Re = oracle.int64_bmm_broadcast(A, W, a_rs, b_rs, c)
    assert np.array_equal(host(C), Ce), "quotient differs"
    assert np.array_equal(host(R), Re), "remainder differs"


@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("c", [0, 29])
def test_gemm_config1_wkv_a(K, oracle, path, c):
    """Benchmark config 1: Y[16,576] = X[16,7168] @ W[576,7168]^T, X in 2^20, W in 2^16, int64 W."""
    rng = np.random.default_rng(1000)
    A = rand_i64(rng, (1, 16, 7168), 20)
    W = rand_i64(rng, (576, 7168), 16)
    _gemm_case(K, oracle, path, A, W, 1, 1, c)


@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("bits_a,bits_w,w32,c", [(37, 31, True, 30), (63, 31, True, 29), (63, 63, False, 0),
                                                 (63, 63, False, 1), (63, 63, False, 29), (63, 63, False, 63),
                                                 (20, 16, False, 33), (31, 31, False, 16), (47, 40, False, 7)])
def test_gemm_ranges_and_shifts(K, oracle, path, bits_a, bits_w, w32, c):
    rng = np.random.default_rng(bits_a * 100 + bits_w + c)
    A = rand_i64(rng, (2, 70, 300), bits_a)
    W = rand_i32(rng, (150, 300), bits_w) if w32 else rand_i64(rng, (150, 300), bits_w)
    if bits_a == 63:
        A[0, 0, :4] = [-(1 << 63), (1 << 63) - 1, 0x7F7F7F7F7F7F7F80, 0x7F7F7F7F7F7F7F7F]
    if bits_w == 63:
        W[0, :4] = [(1 << 63) - 1, -(1 << 63), -0x7F7F7F7F7F7F7F80, 0x7F7F7F7F7F7F7F80]
    _gemm_case(K, oracle, path, A, W, 1, 1, c)


@pytest.mark.parametrize("c", [0, 1, 8, 31, 32, 33, 40, 63])
@pytest.mark.parametrize("bits_a,bits_w,w32", [(63, 63, False), (63, 31, True), (36, 63, False)])
def test_gemm_many_digit_operands_at_every_shift(K, oracle, bits_a, bits_w, w32, c):
    """Operands of up to nine digits: the MFMA path leaves out the digit pairs whose weight lies above the stored bits
    [c, c + 64) of the sum (8, 12 or all diagonals), so shifts on both sides of each boundary are checked, with
    values whose top digits are as large as they get."""
    rng = np.random.default_rng(bits_a + bits_w + c)
    A = rand_i64(rng, (1, 130, 520), bits_a)
    W = rand_i32(rng, (200, 520), bits_w) if w32 else rand_i64(rng, (200, 520), bits_w)
    lim_a, lim_w = (1 << bits_a) - 1, (1 << bits_w) - 1
    A[0, 1, :] = np.where(np.arange(520) % 2 == 0, lim_a, -lim_a - 1)
    W[3, :] = np.where(np.arange(520) % 3 == 0, -lim_w - 1, lim_w)
    for _ in range(3):          # (a first call may run on digits remembered for other operands at these addresses)
        _gemm_case(K, oracle, 2, A, W, 1, 1, c)
    _, la, lb = K.gemm_last_plan()
    kept = 8 if c == 0 else (12 if c <= 32 else 16)
    if (la, lb) == (9, 9):      # the other digit counts have no 12-diagonal instance
        assert K.gemm_last_pairs() == sum(1 for i in range(9) for j in range(9) if i + j < kept)
    elif c == 0:
        assert K.gemm_last_pairs() == sum(1 for i in range(la) for j in range(lb) if i + j < 8)
    K.lib.zk_gemm_set_path(0)


@pytest.mark.parametrize("Kd", [14560, 14600, 16384, 18432])
def test_gemm_long_k_with_nine_digit_operands(K, oracle, Kd):
    """the int32 accumulators of the MFMA path hold min(NA, NB) * K * 2^14: with nine digits that ends at K = 14563.
    Beyond it every tile is split along K (partial sums, then the finishing kernel) instead of falling back to the
    vector ALU; operands whose digits all sit at their extremes, on both sides of the bound and at the model's 16384 /
    18432"""
    rng = np.random.default_rng(Kd)
    A = rand_i64(rng, (1, 70, Kd), 63)
    W = rand_i64(rng, (150, Kd), 63)
    A[0, 0, :] = -0x7F7F7F7F7F7F7F80 - 1            # every digit -128 (and the ninth 0): the largest products
    A[0, 1, :] = 0x7F7F7F7F7F7F7F7F
    W[0, :] = -0x7F7F7F7F7F7F7F80 - 1
    W[1, :] = 0x7F7F7F7F7F7F7F7F
    for c in (0, 29, 63):
        _gemm_case(K, oracle, 2, A, W, 1, 1, c)
        assert K.gemm_last_plan() == (2, 9, 9), "the long K must stay on the MFMA path"
    K.lib.zk_gemm_set_path(0)


@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (1, 1, 7, 1), (3, 5, 17, 9), (1, 64, 64, 64), (1, 65, 129, 63),
                                   (1, 128, 32, 256), (2, 33, 1000, 31), (1, 257, 96, 130)])
def test_gemm_ragged_shapes(K, oracle, path, shape):
    Bd, M, Kd, N = shape
    rng = np.random.default_rng(sum(shape))
    A = rand_i64(rng, (Bd, M, Kd), 40)
    W = rand_i64(rng, (N, Kd), 33)
    _gemm_case(K, oracle, path, A, W, 1, 1, 13)


@pytest.mark.parametrize("bits", [(20, 16), (37, 31), (45, 20)])
@pytest.mark.parametrize("shape", [(1, 8, 512, 2048), (2, 20, 300, 1100), (1, 32, 96, 1024), (1, 3, 2048, 7168),
                                   (1, 100, 2048, 520), (1, 40, 4096, 200)])
def test_gemm_few_rows_many_columns(K, oracle, shape, bits):
    """expert-FFN-like shapes: a handful of tokens against a wide weight matrix (32-row tiles, digit planes of A,
    K split over many workgroups), and mid-sized launches that are split along K as well"""
    Bd, M, Kd, N = shape
    rng = np.random.default_rng(sum(shape) + bits[0])
    A = rand_i64(rng, (Bd, M, Kd), bits[0])
    W = rand_i64(rng, (N, Kd), bits[1])
    for c in (0, 23):
        _gemm_case(K, oracle, 2, A, W, 1, 1, c)
    K.lib.zk_gemm_set_path(0)


@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("shape", [(1, 70, 300, 150), (2, 8, 2048, 512), (1, 300, 1024, 300)])
def test_gemm_without_remainder(K, oracle, path, shape):
    """R = NULL: the quotient is the same and nothing is stored for the remainder (whole tiles, split-K tiles and
    the vector-ALU kernel each have their own epilogue)"""
    Bd, M, Kd, N = shape
    rng = np.random.default_rng(sum(shape))
    A, W = rand_i64(rng, (Bd, M, Kd), 37), rand_i32(rng, (N, Kd), 31)
    K.lib.zk_gemm_set_path(path)
    C, R = K.int64_bmm_broadcast(dev(A), dev(W), 1, 1, 29, want_remainder=False)
    assert R is None
    assert np.array_equal(host(C), oracle.int64_bmm_broadcast(A, W, 1, 1, 29)[0])
    K.lib.zk_gemm_set_path(0)


@pytest.mark.parametrize("path", PATHS)
def test_gemm_operand_divisors(K, oracle, path):
    """head projection divides the weights by 256 (inference/model.py:1519); division truncates toward zero"""
    rng = np.random.default_rng(5)
    A = rand_i64(rng, (1, 9, 200), 45)
    W = rand_i64(rng, (40, 200), 36)
    for a_rs, b_rs in ((1, 256), (3, 1), (-7, 5)):
        _gemm_case(K, oracle, path, A, W, a_rs, b_rs, 21)


@pytest.mark.parametrize("w32", [False, True])
@pytest.mark.parametrize("b_rs", [2, 256, 1 << 20, 1 << 40, 1 << 62])
def test_gemm_head_projection_divisor_on_mfma(K, oracle, w32, b_rs):
    """the head's shape in small: one to a few rows against many columns, weights divided by a power of two before the
    product (inference/model.py:1519).  Truncation toward zero matters for the negative weights; the 32-row MFMA
    kernels fold the division into their digit split, more rows go to the vector-ALU kernel's shift path."""
    rng = np.random.default_rng(b_rs % 1000 + w32)
    W = rand_i32(rng, (700, 320), 31) if w32 else rand_i64(rng, (700, 320), 45)
    W[0, :6] = [-256, -255, -257, 255, 256, -1]
    K.lib.zk_gemm_set_path(0)
    for M in (1, 7, 32, 40):
        A = rand_i64(rng, (1, M, 320), 36)
        for _ in range(2):                                     # the second call runs on the remembered digit counts
            _gemm_case(K, oracle, 0, A, W, 1, b_rs, 21)
        # one or two rows take the matrix-vector kernel, up to 16 the 16-row MFMA tiles (any width: a wavefront that
        # meets more than five digits recomputes on the vector ALU by itself), up to 32 the 32-row MFMA kernels, for
        # which 45-bit weights / 2 still need six digits
        mfma_expected = 2 < M <= 16 or (16 < M <= 32 and (w32 or b_rs >= 256))
        assert (K.gemm_last_plan()[0] == 2) == mfma_expected, (M, K.gemm_last_plan())
    # the MFMA kernels on a single row, asked for by name
    A = rand_i64(rng, (1, 1, 320), 36)
    _gemm_case(K, oracle, 2, A, W, 1, b_rs, 21)
    assert K.gemm_last_plan()[0] == 2
    K.lib.zk_gemm_set_path(0)


@pytest.mark.parametrize("M", [1, 2, 3, 4])
@pytest.mark.parametrize("w32", [False, True])
def test_gemm_one_or_two_rows(K, oracle, M, w32):
    """a decoding step: the matrix-vector kernel (automatic path; three or four rows in two passes) on narrow and wide
    outputs, odd K, unaligned rows, batches, full-range operands, operand divisors and every shift class"""
    rng = np.random.default_rng(40 + M + w32)
    for Bd, Kd, N, bits_a, bits_w, c in ((1, 7168, 576, 20, 16, 29), (1, 1000, 5000, 37, 31, 30), (3, 333, 130, 63, 63, 0),
                                         (1, 1, 1, 63, 63, 63), (2, 4097, 9, 50, 40, 33), (1, 64, 20000, 31, 31, 16)):
        A = rand_i64(rng, (Bd, M, Kd), bits_a)
        W = rand_i32(rng, (N, Kd), bits_w) if w32 else rand_i64(rng, (N, Kd), bits_w)
        _gemm_case(K, oracle, 0, A, W, 1, 1, c)
        assert K.gemm_last_plan()[0] == 1
    A, W = rand_i64(rng, (1, M, 300), 45), (rand_i32(rng, (77, 300)) if w32 else rand_i64(rng, (77, 300), 50))
    for a_rs, b_rs in ((1, 256), (3, 1), (-7, 5), (1 << 20, 1 << 3)):
        _gemm_case(K, oracle, 0, A, W, a_rs, b_rs, 21)
    # the per-head einsums of a decoding step: M rows per head, the heads as a strided batch
    H, D, Cc = 16, 24, 40
    a = rand_i64(rng, (1, M, H, Cc), 30)
    w = rand_i32(rng, (H, D, Cc), 25)
    assert np.array_equal(host(K.einsum_bshc_hdc_bshd(dev(a), dev(w), 21)), oracle.einsum_bshc_hdc_bshd(a, w, 21))
    assert K.gemm_last_plan()[0] == 1
    q = rand_i64(rng, (1, M, H, D), 30)
    assert np.array_equal(host(K.einsum_bshd_hdc_bshc(dev(q), dev(w), 21)), oracle.einsum_bshd_hdc_bshc(q, w, 21))
    assert K.gemm_last_plan()[0] == 1
    # rows of A that start 8 bytes off a 16-byte boundary: the element-wise loads
    buf = torch.zeros((M * 301 + 1,), dtype=torch.int64, device="cuda")
    Av = rand_i64(rng, (1, M, 301), 40)
    Ad = buf[1:].view(1, M, 301)
    Ad.copy_(dev(Av))
    Wv = rand_i32(rng, (50, 301)) if w32 else rand_i64(rng, (50, 301), 40)
    Wd = dev(Wv)
    C = torch.empty((1, M, 50), dtype=torch.int64, device="cuda")
    R = torch.empty_like(C)
    fn = K.lib.int64_32_bmm_broadcast_launcher if w32 else K.lib.int64_64_bmm_broadcast_launcher
    fn(Ad.data_ptr(), Wd.data_ptr(), C.data_ptr(), R.data_ptr(), 1, 1, 17, 1, M, 301, 50)
    torch.cuda.synchronize()
    K._check("gemv")
    Ce, Re = oracle.int64_bmm_broadcast(Av, Wv, 1, 1, 17)
    assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)


@pytest.mark.parametrize("w32", [False, True])
@pytest.mark.parametrize("M", [1, 3, 8, 15, 16])
def test_gemm_up_to_16_rows(K, oracle, M, w32):
    """the 16-row MFMA tiles (every wavefront on its own, digit counts taken from each step's data): one K slice and
    several (every slice writes its partial sums into a slot of its own, a second launch adds the slots), ragged N and K, batches, every digit path from
    (3,3) to (5,5), operands beyond five digits (the wavefronts that meet them recompute on the vector ALU), widths that
    change from step to step, every shift class, with and without remainder"""
    rng = np.random.default_rng(160 + M + w32)
    K.lib.zk_gemm_set_path(2)
    for Bd, Kd, N, bits_a, bits_w, c in ((1, 7168, 576, 20, 16, 29), (1, 2048, 7168, 28, 31, 30), (2, 333, 130, 37, 30, 0),
                                         (1, 64, 20000, 31, 31, 16), (3, 1000, 50, 63, 63, 0), (1, 4100, 33, 63, 31, 63),
                                         (1, 1, 1, 63, 63, 1), (1, 640, 700, 45, 20, 33), (5, 130, 31, 22, 22, 7)):
        A = rand_i64(rng, (Bd, M, Kd), bits_a)
        W = rand_i32(rng, (N, Kd), min(bits_w, 31)) if w32 else rand_i64(rng, (N, Kd), bits_w)
        _gemm_case(K, oracle, 2, A, W, 1, 1, c)
        assert K.gemm_last_plan() == (2, 0, 0)
    # widths that differ from step to step and from column tile to column tile: narrow everywhere, four and five digits
    # in places, and one element beyond five digits in a single step of a single row
    Kd, N = 1024, 200
    A = rand_i64(rng, (1, M, Kd), 20)
    W = rand_i32(rng, (N, Kd), 16) if w32 else rand_i64(rng, (N, Kd), 16)
    A[0, :, 128:192] = rand_i64(rng, (M, 64), 29)
    A[0, M - 1, 300] = -(1 << 37)
    W[40:56, 512:640] = (rand_i32(rng, (16, 128), 31) if w32 else rand_i64(rng, (16, 128), 37))
    _gemm_case(K, oracle, 2, A, W, 1, 1, 23)
    A[0, 0, 1000] = (1 << 62) + 12345
    if not w32:
        W[199, 7] = -(1 << 63)
    _gemm_case(K, oracle, 2, A, W, 1, 1, 23)
    # no remainder wanted; operand divisor on B
    C, R = K.int64_bmm_broadcast(dev(A), dev(W), 1, 1, 23, want_remainder=False)
    assert R is None and np.array_equal(host(C), oracle.int64_bmm_broadcast(A, W, 1, 1, 23)[0])
    _gemm_case(K, oracle, 2, A, W, 1, 256, 11)
    # digits at their extremes over many steps between two folds of the int32 accumulators
    # (digits -128, -128, -128, -128, 63: the largest magnitudes among the values that take the five-digit path)
    x5 = (63 << 32) - 0x80808080
    A = np.full((1, M, 2048), x5, np.int64)
    W = np.full((70, 2048), -(1 << 31), np.int32) if w32 else np.full((70, 2048), x5, np.int64)
    W[1::2] = (1 << 31) - 1 if w32 else -x5
    _gemm_case(K, oracle, 2, A, W, 1, 1, 40)
    # rows that start 8 bytes off a 16-byte boundary: the element-wise loads
    buf = torch.zeros((M * 301 + 1,), dtype=torch.int64, device="cuda")
    Av = rand_i64(rng, (1, M, 301), 30)
    Ad = buf[1:].view(1, M, 301)
    Ad.copy_(dev(Av))
    Wv = rand_i32(rng, (50, 301)) if w32 else rand_i64(rng, (50, 301), 30)
    Wd = dev(Wv)
    C = torch.empty((1, M, 50), dtype=torch.int64, device="cuda")
    R = torch.empty_like(C)
    fn = K.lib.int64_32_bmm_broadcast_launcher if w32 else K.lib.int64_64_bmm_broadcast_launcher
    fn(Ad.data_ptr(), Wd.data_ptr(), C.data_ptr(), R.data_ptr(), 1, 1, 17, 1, M, 301, 50)
    K._check("rows16")
    Ce, Re = oracle.int64_bmm_broadcast(Av, Wv, 1, 1, 17)
    assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
    # the per-head einsums on a few sequence positions: the heads as a strided batch of k-contiguous int32 matrices
    H, D, Cc = 16, 24, 40
    a = rand_i64(rng, (1, M, H, Cc), 30)
    w = rand_i32(rng, (H, D, Cc), 25)
    assert np.array_equal(host(K.einsum_bshc_hdc_bshd(dev(a), dev(w), 21)), oracle.einsum_bshc_hdc_bshd(a, w, 21))
    assert K.gemm_last_plan() == (2, 0, 0)
    # and the scores of a few positions against a cache: bshc,btc->bsht with S * H <= 16
    qq = rand_i64(rng, (2, 1, M, 192), 30)
    kk = rand_i64(rng, (2, 300, 192), 24)
    assert np.array_equal(host(K.einsum_bshc_btc_bsht(dev(qq), dev(kk), 21)), oracle.einsum_bshc_btc_bsht(qq, kk, 21))
    K.lib.zk_gemm_set_path(0)


def test_gemm_split_k_slots_of_an_earlier_call_do_not_show_through(K, oracle):
    """the K slices of a call write partial sums into slots that the library keeps between calls, and nothing clears
    them: calls of different shapes one after the other, asynchronously (a larger one before a smaller one, the same
    one twice), must each add up their own slots only"""
    rng = np.random.default_rng(170)
    K.lib.zk_gemm_set_path(2)
    shapes = [(16, 7168, 576), (5, 4096, 64), (16, 7168, 576), (9, 2048, 1000), (3, 8192, 33)]
    ops = [(rand_i64(rng, (1, M, Kd), 30), rand_i64(rng, (N, Kd), 33)) for M, Kd, N in shapes]
    devs = [(dev(a), dev(w)) for a, w in ops]
    outs = [K.int64_bmm_broadcast(a, w, 1, 1, 19) for a, w in devs for _ in range(2)]
    for i, (a, w) in enumerate(ops):
        Ce, Re = oracle.int64_bmm_broadcast(a, w, 1, 1, 19)
        for C, R in outs[2 * i: 2 * i + 2]:
            assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re), shapes[i]
    K.lib.zk_gemm_set_path(0)


@pytest.mark.parametrize("M", [1, 2])
def test_gemm_rows_staged_in_lds(K, oracle, M):
    """one or two rows against int32 weights with K % 4 == 0 and a wide output: the kernel that stages the rows in LDS as
    three 21-bit pieces (several staging rounds, one, two and four columns per wave with ragged last workgroups, strided
    batches, shifts 0 and 63, and the operands that bring its 64-bit accumulators closest to their limit)"""
    rng = np.random.default_rng(70 + M)
    for Bd, Kd, N, bits_a, c in ((1, 9000, 2100, 63, 29), (1, 520, 16390, 40, 0), (1, 516, 9001, 63, 63), (3, 512, 900, 31, 17),
                                 (1, 256, 3000, 63, 31)):
        A = rand_i64(rng, (Bd, M, Kd), bits_a)
        W = rand_i32(rng, (N, Kd), 31)
        A[0, 0, :3] = [-(1 << 63), (1 << 63) - 1, -1]
        W[0, :3] = [-(1 << 31), (1 << 31) - 1, -(1 << 31)]
        _gemm_case(K, oracle, 0, A, W, 1, 1, c)
        assert K.gemm_last_plan()[0] == 1
    # the longest K it takes, every product at its largest magnitude and of one sign per column
    Kd, N = 65536, 2048
    A = np.full((1, M, Kd), -(1 << 63), np.int64)
    A[0, M - 1, 1::2] = (1 << 63) - 1
    W = np.full((N, Kd), -(1 << 31), np.int32)
    W[1::2] = (1 << 31) - 1
    W[2, ::3] = 12345
    _gemm_case(K, oracle, 0, A, W, 1, 1, 33)
    assert K.gemm_last_plan()[0] == 1


@pytest.mark.parametrize("bits_w", [16, 28, 36, 63, -16, -30, -31])
def test_gemm_prepared_weights(K, oracle, bits_w):
    """int64 weights split into digit planes once (zk_gemm_prepare_weights): the same bits as the unprepared call on
    32-row and full tiles, ragged N and K, split K, few rows, activations that need more digits than any kernel with the
    planes' digit count has (the call then splits the original weights), weights changed and prepared again, release"""
    w32, bits_w = bits_w < 0, abs(bits_w)                # negative: int32 weights of that many bits
    rng = np.random.default_rng(bits_w + w32)
    for M, Kd, N, bits_a, c in ((16, 7168, 576, 20, 29), (130, 300, 150, 20, 0), (512, 1000, 700, 23, 29), (3, 333, 77, 30, 33),
                                (1, 520, 300, 20, 23), (70, 96, 2100, 63, 31)):
        A = rand_i64(rng, (2, M, Kd), bits_a)
        W = rand_i32(rng, (N, Kd), bits_w) if w32 else rand_i64(rng, (N, Kd), bits_w)
        W[0, :2] = [-(1 << bits_w), (1 << bits_w) - 1]
        Ce, Re = oracle.int64_bmm_broadcast(A, W, 1, 1, c)
        Ad, Wd = dev(A), dev(W)
        K.prepare_weights(Wd)
        for rep in range(2):
            C, R = K.int64_bmm_broadcast(Ad, Wd, 1, 1, c)
            assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re), (M, Kd, N, bits_a, c, rep)
        if bits_a <= 23 and bits_w <= 36 and M > 4:
            assert K.lib.zk_gemm_last_prepared() == 1            # the planes were used
        # other weights under the same pointer, prepared again
        W2 = rand_i32(rng, (N, Kd), 12) if w32 else rand_i64(rng, (N, Kd), 12)
        Wd.copy_(dev(W2))
        K.prepare_weights(Wd)
        C, R = K.int64_bmm_broadcast(Ad, Wd, 1, 1, c)
        Ce2, Re2 = oracle.int64_bmm_broadcast(A, W2, 1, 1, c)
        assert np.array_equal(host(C), Ce2) and np.array_equal(host(R), Re2), ("again", M, Kd, N)
        K.release_weights(Wd)
        C, R = K.int64_bmm_broadcast(Ad, Wd, 1, 1, c)
        assert np.array_equal(host(C), Ce2) and np.array_equal(host(R), Re2), ("released", M, Kd, N)
        assert K.lib.zk_gemm_last_prepared() == 0


def test_gemm_prepared_weights_pipelined_kernel(K, oracle):
    """three digits a side with planes for both operands run on the software-pipelined 128 x 128 kernel (loads through a
    ring of LDS stages, the next step's fragments read beside the MFMAs): several rounds of tiles with the last one cut
    along K, a K that is not a whole step and one shorter than the ring is deep, two batches, ragged M and N, int32
    weights, a K beyond one pass of the int32 accumulators (every tile cut), C alone"""
    rng = np.random.default_rng(77)
    keep = []
    for (Bd, M, N, Kd, bits_a, bits_w, w32, c) in ((1, 640, 6656, 2048, 20, 16, False, 17), (1, 512, 8192, 96, 20, 16, False, 0),
                                                   (1, 600, 6700, 227, 21, 16, False, 23), (2, 384, 5632, 160, 20, 16, False, 9),
                                                   (1, 640, 6656, 1024, 20, 16, True, 17), (1, 130, 200, 40, 21, 16, False, 23),
                                                   (1, 130, 256, 50000, 20, 16, False, 29), (1, 1100, 33000, 100, 20, 16, False, 29)):
        A = rand_i64(rng, (Bd, M, Kd), bits_a)
        W = rand_i32(rng, (N, Kd), bits_w) if w32 else rand_i64(rng, (N, Kd), bits_w)
        Ce, Re = oracle.int64_bmm_broadcast(A, W, 1, 1, c)
        Ad, Wd = dev(A), dev(W)
        keep.append(Wd)
        K.prepare_weights(Wd)
        try:
            for rep in range(3):            # (the first call may run on a guess made for other activations at this address)
                before = K.lib.zk_gemm_pipe_calls()
                C, R = K.int64_bmm_broadcast(Ad, Wd, 1, 1, c)
                assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re), (Bd, M, N, Kd, w32, c, rep)
            assert K.gemm_last_plan()[1:] == (3, 3) and K.lib.zk_gemm_last_prepared() == 1
            assert K.lib.zk_gemm_pipe_calls() == before + 1, (Bd, M, N, Kd)
            C, R = K.int64_bmm_broadcast(Ad, Wd, 1, 1, c, want_remainder=False)
            assert R is None and np.array_equal(host(C), Ce)
        finally:
            K.release_weights(Wd)


@pytest.mark.parametrize("w32", [False, True])
@pytest.mark.parametrize("T,Kr", [(1, 8), (40, 3), (300, 4)])
def test_grouped_bmm_prepared_weights(K, oracle, T, Kr, w32):
    """the experts' weights prepared through their pointer table: one launch over all experts on the planes, the same
    bits as without; wide activations fall back to splitting the original weights"""
    rng = np.random.default_rng(T + Kr)
    E, Kd, N = 16, 200, 300
    idx = _routing(rng, T, E, Kr)
    ws = [rand_i32(rng, (N, Kd), 30) if w32 else rand_i64(rng, (N, Kd), 16) for _ in range(E)]
    wd = [dev(w) for w in ws]
    tab = K.pointer_table(wd)
    K.prepare_weights(tab, groups=E, N=N, K=Kd, b32=w32)
    d = K.moe_dispatch(dev(idx), E)
    seg, tok, _ = oracle.moe_dispatch(idx, E)
    for bits_a in (20, 45):
        x = rand_i64(rng, (T, Kd), bits_a)
        xs = K.moe_gather_rows(dev(x), d)
        before = K.lib.zk_gemm_grouped_mfma_calls()
        for c in (0, 19):
            C, R = K.int64_grouped_bmm(xs, tab, w32, N, c, d, want_remainder=True)
            Ce, Re = oracle.grouped_bmm(x[tok], ws, seg, c)
            assert np.array_equal(host(C), Ce), ("quotient", bits_a, c)
            assert np.array_equal(host(R), Re), ("remainder", bits_a, c)
        if bits_a == 20 and T * Kr > (64 if w32 else 32):
            assert K.lib.zk_gemm_grouped_mfma_calls() - before == 2 and K.lib.zk_gemm_last_prepared() == 1
    K.release_weights(tab)
    C = K.int64_grouped_bmm(xs, tab, w32, N, 19, d)
    assert np.array_equal(host(C), oracle.grouped_bmm(x[tok], ws, seg, 19)[0])


def test_gemm_rejects_bad_arguments(K):
    A = torch.zeros((1, 2, 3), dtype=torch.int64, device="cuda")
    W = torch.zeros((4, 3), dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError):
        K.int64_bmm_broadcast(A, W, 1, 1, 64)
    with pytest.raises(RuntimeError):
        K.int64_bmm_broadcast(A, W, 0, 1, 3)
    assert K.lib.zk_last_error() == 0          # the wrapper clears the channel after raising


@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("full_range", [False, True])
def test_gemm_config4_full_size_sampled(K, oracle, path, full_range):
    """Benchmark config 4 at full size: 512 x 7168 against W[18432,7168].  The oracle checks a sample of rows and
    columns exactly; linearity in A (at shift 0, where the result is the wrapping int64 product) covers the rest."""
    if path == 1 and full_range:
        pytest.skip("one full-size VALU run is enough")
    g = torch.Generator(device="cpu").manual_seed(4000 + int(full_range))
    M, Kd, N = 512, 7168, 18432
    if full_range:
        A = torch.randint(-(1 << 63), (1 << 63) - 1, (1, M, Kd), generator=g, dtype=torch.int64)
        W = torch.randint(-(1 << 63), (1 << 63) - 1, (N, Kd), generator=g, dtype=torch.int64)
    else:
        A = torch.randint(-(1 << 20), 1 << 20, (1, M, Kd), generator=g, dtype=torch.int64)
        W = torch.randint(-(1 << 16), 1 << 16, (N, Kd), generator=g, dtype=torch.int64)
    K.lib.zk_gemm_set_path(path)
    Ad, Wd = A.cuda(), W.cuda()
    c = 29
    C, R = K.int64_bmm_broadcast(Ad, Wd, 1, 1, c)
    rows = torch.tensor([0, 1, 63, 64, 255, 256, 300, 511])
    cols = torch.cat([torch.arange(0, 40), torch.arange(9000, 9040), torch.arange(N - 48, N)])
    Ce, Re = oracle.int64_bmm_broadcast(A[:, rows].numpy(), W[cols].numpy(), 1, 1, c)
    assert np.array_equal(host(C[:, rows][:, :, cols]), Ce)
    assert np.array_equal(host(R[:, rows][:, :, cols]), Re)
    if not full_range:
        # nothing overflows here: quotient and remainder must rebuild torch's int64 product everywhere
        full = torch.matmul(A[0, :64], W[:2048].T)          # torch's CPU int64 matmul: the reference's CPU path
        assert torch.equal((C[0, :64, :2048] * (1 << c) + R[0, :64, :2048]).cpu(), full)
    # linearity at shift 0: (A1 + A2) W = A1 W + A2 W  (mod 2^64)
    A2 = torch.roll(Ad, 1, dims=1)
    C0, _ = K.int64_bmm_broadcast(Ad, Wd, 1, 1, 0)
    C1, _ = K.int64_bmm_broadcast(A2, Wd, 1, 1, 0)
    C2, _ = K.int64_bmm_broadcast(Ad + A2, Wd, 1, 1, 0)
    assert torch.equal(C2, C0 + C1)
    assert torch.equal(C1, torch.roll(C0, 1, dims=1))
    # shift 0 is the product modulo 2^64, and torch's CPU int64 matmul (the reference's CPU path) wraps the same way:
    # a block of rows and columns is compared with it directly, full-range operands included
    assert torch.equal(C0[0, 100:148, 4000:5024].cpu(), torch.matmul(A[0, 100:148], W[4000:5024].T))


@pytest.mark.parametrize("seed", range(40 * SEEDS))
def test_gemm_seeded_random_problems(K, oracle, seed):
    """a sweep no hand-picked list would make: random batch, shape, operand widths, weight type and shift per case, on
    the MFMA path (whole tiles, edge tiles, 32-row tiles, K split, digit planes or not, few or many diagonals kept)"""
    rng = np.random.default_rng(9000 + seed)
    for _ in range(6):
        Bd = int(rng.choice([1, 1, 2, 3]))
        M = int(rng.choice([1, 5, 16, 31, 33, 64, 100, 129, 200, 300]))
        Kd = int(rng.choice([1, 7, 32, 33, 96, 250, 512, 1000, 2048]))
        N = int(rng.choice([1, 9, 64, 127, 130, 256, 520, 1100]))
        while Bd * M * Kd * N > 60_000_000:         # keep the scalar oracle to a fraction of a second per case
            Kd = max(1, Kd // 2)
        w32 = bool(rng.integers(0, 2))
        bits_a = int(rng.choice([3, 12, 20, 31, 37, 47, 56, 63]))
        bits_w = int(rng.choice([3, 12, 16, 24, 31])) if w32 else int(rng.choice([3, 16, 24, 33, 47, 63]))
        c = int(rng.choice([0, 1, 8, 16, 23, 29, 31, 32, 33, 40, 63]))
        A = rand_i64(rng, (Bd, M, Kd), bits_a)
        W = rand_i32(rng, (N, Kd), bits_w) if w32 else rand_i64(rng, (N, Kd), bits_w)
        try:
            _gemm_case(K, oracle, 2, A, W, 1, 1, c)
        except AssertionError as e:
            raise AssertionError("%s for B=%d M=%d K=%d N=%d w32=%s bits=(%d,%d) c=%d" % (e, Bd, M, Kd, N, w32, bits_a, bits_w, c))
    K.lib.zk_gemm_set_path(0)


@pytest.mark.parametrize("seed", range(20 * SEEDS))
def test_einsums_seeded_random_problems(K, oracle, seed):
    """the four einsums on random shapes and operand widths (strided A rows, k-major and int32 B, per-head batches)"""
    rng = np.random.default_rng(9500 + seed)
    for _ in range(3):
        B = int(rng.choice([1, 2]))
        S = int(rng.choice([1, 7, 40, 130]))
        H = int(rng.choice([1, 3, 16]))
        D = int(rng.choice([8, 24, 64, 128]))
        Cc = int(rng.choice([16, 40, 64, 192, 512]))
        T = int(rng.choice([1, 33, 70, 256, 300]))
        while B * S * H * max(D * Cc, T * Cc) > 40_000_000:
            S = max(1, S // 2)
        bits = int(rng.choice([10, 20, 30, 40, 63]))
        rescale = int(rng.choice([0, 19, 21, 23, 29, 37]))
        q = rand_i64(rng, (B, S, H, D), bits)
        w1 = rand_i32(rng, (H, D, Cc), int(rng.choice([8, 25, 31])))
        a = rand_i64(rng, (B, S, H, Cc), bits)
        kv = rand_i64(rng, (B, T, Cc), int(rng.choice([10, 24, 40])))
        pr = rand_i64(rng, (B, S, H, T), int(rng.choice([19, 30])))
        tag = "B=%d S=%d H=%d D=%d C=%d T=%d bits=%d rescale=%d" % (B, S, H, D, Cc, T, bits, rescale)
        assert np.array_equal(host(K.einsum_bshd_hdc_bshc(dev(q), dev(w1), rescale)), oracle.einsum_bshd_hdc_bshc(q, w1, rescale)), tag
        assert np.array_equal(host(K.einsum_bshc_btc_bsht(dev(a), dev(kv), rescale)), oracle.einsum_bshc_btc_bsht(a, kv, rescale)), tag
        assert np.array_equal(host(K.einsum_bsht_btc_bshc(dev(pr), dev(kv), rescale)), oracle.einsum_bsht_btc_bshc(pr, kv, rescale)), tag
        assert np.array_equal(host(K.einsum_bshc_hdc_bshd(dev(a), dev(w1), rescale)), oracle.einsum_bshc_hdc_bshd(a, w1, rescale)), tag


# ---------------------------------------------------------------------------------- einsums -----
@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("bits", [20, 40, 63])
def test_einsums(K, oracle, path, bits):
    K.lib.zk_gemm_set_path(path)
    rng = np.random.default_rng(bits)
    B, S, H, D, Cc, T = 2, 9, 5, 24, 40, 70
    q = rand_i64(rng, (B, S, H, D), bits)
    w1 = rand_i32(rng, (H, D, Cc))
    a = rand_i64(rng, (B, S, H, Cc), bits)
    kv = rand_i64(rng, (B, T, Cc), bits)
    p = rand_i64(rng, (B, S, H, T), bits)
    w2 = rand_i32(rng, (H, D, Cc))
    for rescale in (0, 21, 23, 37):
        assert np.array_equal(host(K.einsum_bshd_hdc_bshc(dev(q), dev(w1), rescale)),
                              oracle.einsum_bshd_hdc_bshc(q, w1, rescale))
        assert np.array_equal(host(K.einsum_bshc_btc_bsht(dev(a), dev(kv), rescale)),
                              oracle.einsum_bshc_btc_bsht(a, kv, rescale))
        assert np.array_equal(host(K.einsum_bsht_btc_bshc(dev(p), dev(kv), rescale)),
                              oracle.einsum_bsht_btc_bshc(p, kv, rescale))
        assert np.array_equal(host(K.einsum_bshc_hdc_bshd(dev(a), dev(w2), rescale)),
                              oracle.einsum_bshc_hdc_bshd(a, w2, rescale))


@pytest.mark.parametrize("path", PATHS)
def test_einsums_model_shapes(K, oracle, path):
    """MLA absorb shapes at a short prefill: H=128, nope 128, kv_lora 512, rope 64 (inference/model.py:862-951)."""
    K.lib.zk_gemm_set_path(path)
    rng = np.random.default_rng(77)
    B, S, H, T = 1, 4, 128, 12
    q_nope = rand_i64(rng, (B, S, H, 128), 24)
    wkv_b_1 = rand_i32(rng, (H, 128, 512), 28)
    qn = K.einsum_bshd_hdc_bshc(dev(q_nope), dev(wkv_b_1), 33)
    assert np.array_equal(host(qn), oracle.einsum_bshd_hdc_bshc(q_nope, wkv_b_1, 33))
    kvc = rand_i64(rng, (B, T, 512), 26)
    s1 = K.einsum_bshc_btc_bsht(qn, dev(kvc), 23)
    assert np.array_equal(host(s1), oracle.einsum_bshc_btc_bsht(host(qn), kvc, 23))
    q_pe = rand_i64(rng, (B, S, H, 64), 22)
    pec = rand_i64(rng, (B, T, 64), 24)
    s2 = K.einsum_bshc_btc_bsht(dev(q_pe), dev(pec), 21)
    assert np.array_equal(host(s2), oracle.einsum_bshc_btc_bsht(q_pe, pec, 21))
    P = rand_i64(rng, (B, S, H, T), 19)
    o = K.einsum_bsht_btc_bshc(dev(P), dev(kvc), 23)
    assert np.array_equal(host(o), oracle.einsum_bsht_btc_bshc(P, kvc, 23))
    wkv_b_2 = rand_i32(rng, (H, 128, 512), 28)
    x = K.einsum_bshc_hdc_bshd(o, dev(wkv_b_2), 31)
    assert np.array_equal(host(x), oracle.einsum_bshc_hdc_bshd(host(o), wkv_b_2, 31))


def test_empty_operands(K, oracle):
    """operands without elements, as torch hands them over (null data pointers): no rows, columns or batches is a call
    that does nothing; an empty contraction leaves the rounding term shifted in every output, as the reference's loop
    over no elements does (int64_gemm.cu:44-78), for the two products, the einsums and the grouped launch; softmax,
    activations, RMSNorm, RoPE and the dispatch of no tokens return without an error"""
    z = lambda *shape, dtype=torch.int64: torch.zeros(shape, dtype=dtype, device="cuda")
    ones = lambda *shape: torch.ones(shape, dtype=torch.int64, device="cuda")
    for A, W in ((z(1, 0, 64), ones(8, 64)), (ones(1, 4, 64), z(0, 64)), (z(0, 4, 64), ones(8, 64))):
        C, R = K.int64_bmm_broadcast(A, W, 1, 1, 3)
        assert C.numel() == 0 and R.numel() == 0
    for path in (0, 1, 2):
        K.lib.zk_gemm_set_path(path)
        try:
            for M, N, w32, c in ((4, 8, False, 3), (200, 300, False, 0), (5, 7, True, 63), (16, 576, True, 17)):
                C = torch.full((2, M, N), 77, dtype=torch.int64, device="cuda")
                R = torch.full((2, M, N), 77, dtype=torch.int64, device="cuda")
                A, W = z(2, M, 0), z(N, 0, dtype=torch.int32 if w32 else torch.int64)
                fn = K.lib.int64_32_bmm_broadcast_launcher if w32 else K.lib.int64_64_bmm_broadcast_launcher
                fn(A.data_ptr(), W.data_ptr(), C.data_ptr(), R.data_ptr(), 1, 1, c, 2, M, 0, N)
                K._check("bmm with K = 0")
                Ce, Re = oracle.int64_bmm_broadcast(np.zeros((2, M, 0), np.int64), np.zeros((N, 0), np.int64), 1, 1, c)
                assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re), (path, M, N, w32, c)
        finally:
            K.lib.zk_gemm_set_path(0)
    for rescale in (0, 1, 7, 40):
        o = K.einsum_bshd_hdc_bshc(z(1, 2, 3, 0), z(3, 0, 5, dtype=torch.int32), rescale)
        assert np.array_equal(host(o), oracle.einsum_bshd_hdc_bshc(np.zeros((1, 2, 3, 0), np.int64), np.zeros((3, 0, 5), np.int32), rescale))
        o = K.einsum_bshc_btc_bsht(z(1, 2, 3, 0), z(1, 4, 0), rescale)
        assert np.array_equal(host(o), oracle.einsum_bshc_btc_bsht(np.zeros((1, 2, 3, 0), np.int64), np.zeros((1, 4, 0), np.int64), rescale))
        o = K.einsum_bsht_btc_bshc(z(1, 2, 3, 0), z(1, 0, 8), rescale)
        assert np.array_equal(host(o), oracle.einsum_bsht_btc_bshc(np.zeros((1, 2, 3, 0), np.int64), np.zeros((1, 0, 8), np.int64), rescale))
        o = K.einsum_bshc_hdc_bshd(z(1, 2, 3, 0), z(3, 6, 0, dtype=torch.int32), rescale)
        assert np.array_equal(host(o), oracle.einsum_bshc_hdc_bshd(np.zeros((1, 2, 3, 0), np.int64), np.zeros((3, 6, 0), np.int32), rescale))
    assert K.einsum_bshc_btc_bsht(ones(1, 2, 3, 8), z(1, 0, 8), 7).shape == (1, 2, 3, 0)
    # the grouped launch over an empty contraction
    idx = dev(np.array([[0, 2], [1, 2], [2, 0]], dtype=np.int64))
    d = K.moe_dispatch(idx, 4)
    ws = [z(6, 0, dtype=torch.int32) for _ in range(4)]
    table = torch.tensor([0x1000 * (i + 1) for i in range(4)], dtype=torch.int64, device="cuda")   # (never dereferenced)
    del ws
    C, R = K.int64_grouped_bmm(z(6, 0), table, True, 6, 5, d, want_remainder=True)
    assert not host(C).any() and not host(R).any()
    # the kernels that are no products
    K.softmax_init_q19(); K.softmax_init_q21(); K.silu_init_q23(); K.silu_init_q25()
    for fn, shape in ((K.softmax_q19, (1, 0, 4, 16)), (K.softmax_q19, (1, 2, 4, 0)), (K.softmax_q21, (0, 2, 4, 16)),
                      (K.silu_q23, (1, 0, 16)), (K.sigmoid_q23, (0, 3, 16)), (K.silu_q25, (2, 3, 0)), (K.sigmoid_q25, (1, 0, 0))):
        Rz = z(*shape)
        fn(Rz, torch.empty_like(Rz))
    out, _ = K.RMS_Norm_int64(z(0, 64), ones(64), 10, 64)
    assert out.shape == (0, 64)
    assert K.complex_int64_mul_broadcast(z(1, 0, 4, 8, 2), z(0, 8, 2)).numel() == 0
    d0 = K.moe_dispatch(z(0, 8), 16)
    assert int(d0["ntiles"].item()) == 0 and not host(d0["seg"]).any()


# ---------------------------------------------------------------------------------- softmax -----
def test_einsum_values_rewritten_with_contiguous_rows(K, oracle, monkeypatch):
    """`bsht,btc->bshc` on the MFMA path copies a small n-contiguous int64 B into row-major scratch first (products of
    2^32 MACs and more; the threshold is lowered here): ragged T and C, two batches, and a second call with another B
    through the same scratch"""
    monkeypatch.setenv("ZK_B_ROWS_MIN_MACS", "1")
    K.lib.zk_reload_env()           # the switches are read when the library is loaded, not per call
    rng = np.random.default_rng(77)
    K.lib.zk_gemm_set_path(2)
    try:
        for Bq, S, H, T, Cc in ((2, 9, 5, 70, 45), (1, 40, 3, 33, 130), (1, 3, 16, 257, 64)):
            for rep in range(2):
                pr = rng.integers(0, 1 << 19, size=(Bq, S, H, T), dtype=np.int64)
                kv = rand_i64(rng, (Bq, T, Cc), 36 if rep else 24)
                assert np.array_equal(host(K.einsum_bsht_btc_bshc(dev(pr), dev(kv), 23)), oracle.einsum_bsht_btc_bshc(pr, kv, 23)), (Bq, S, H, T, Cc, rep)
                assert K.gemm_last_plan()[0] == 2
    finally:
        K.lib.zk_gemm_set_path(0)
        monkeypatch.delenv("ZK_B_ROWS_MIN_MACS")
        K.lib.zk_reload_env()


def _scores(rng, shape, Q, masked=True):
    x = rng.integers(-(12 << Q), 12 << Q, size=shape, dtype=np.int64)
    if masked and shape[-1] > 1:
        T = shape[-1]
        cut = rng.integers(1, T + 1, size=shape[:-1])
        x = np.where(np.arange(T) < cut[..., None], x, x - (1 << 42))       # causal-mask value -(64 << 36)
    return x


@pytest.mark.parametrize("fn,Q", [("softmax_q19", 19), ("softmax_q21", 21)])
@pytest.mark.parametrize("T", [1, 2, 3, 7, 64, 100, 127, 128, 129, 256, 257, 1000, 1024, 1025, 2048, 2049, 5000])
def test_softmax_lengths(K, oracle, fn, Q, T):
    rng = np.random.default_rng(T + Q)
    x = _scores(rng, (1, 3, 5, T), Q)
    R = dev(x)
    C = torch.empty_like(R)
    getattr(K, fn)(R, C)
    Ce, _ = getattr(oracle, fn)(x)
    assert np.array_equal(host(C), Ce)
    assert np.array_equal(host(R), x), "input must stay intact by default"


@pytest.mark.parametrize("fn", ["softmax_q19", "softmax_q21"])
@pytest.mark.parametrize("T", [96, 1024, 3001])
def test_softmax_reference_clobber_mode(K, oracle, fn, T):
    """with the switch on, the input buffer ends up holding the weights, as after the reference's kernel"""
    rng = np.random.default_rng(T)
    x = _scores(rng, (2, 2, 4, T), 19)
    R = dev(x)
    C = torch.empty_like(R)
    K.lib.zk_softmax_clobber_input(1)
    try:
        getattr(K, fn)(R, C)
    finally:
        K.lib.zk_softmax_clobber_input(0)
    Ce, We = getattr(oracle, fn)(x)
    assert np.array_equal(host(C), Ce)
    assert np.array_equal(host(R), We)


@pytest.mark.parametrize("fn", ["softmax_q19", "softmax_q21"])
def test_softmax_hostile_inputs(K, oracle, fn):
    """full-range scores and an arbitrary table: the slow exact paths must agree with the oracle's fixed semantics"""
    rng = np.random.default_rng(9)
    x = rand_i64(rng, (1, 2, 6, 333), 63)
    x[0, 0, 0, :] = 7
    x[0, 0, 1, :] = -(1 << 63)
    lut = rand_i64(rng, (256,), 63)
    for table in (None, lut):
        R = dev(x)
        C = torch.empty_like(R)
        t = dev(table) if table is not None else (K.EXP2_FRAC_LUT_Q19 if fn == "softmax_q19" else K.EXP2_FRAC_LUT_Q21)
        getattr(K.lib, fn)(R.data_ptr(), C.data_ptr(), t.data_ptr(), 1, 2, 6, 333)
        torch.cuda.synchronize()
        Ce, _ = getattr(oracle, fn)(x, table)
        assert np.array_equal(host(C), Ce)


def test_softmax_and_activation_hand_worked_literals(K):
    """the results worked by hand from the reference's source (the steps are written out in test_oracle_pins.py:
    softmax q19 :700-740 and q21 :624-657 of inference/int64_gemm.cu, sigmoid/SiLU q23 :932-946 and q25 :804-818),
    asked of the device library directly: no oracle in between"""
    def smx(fn, row):
        R = dev(np.array(row, np.int64).reshape(1, 1, 1, -1))
        C = torch.empty_like(R)
        getattr(K, fn)(R, C)
        return host(C).ravel().tolist()

    def act(fn, vals):
        R = dev(np.array(vals, np.int64).reshape(1, 1, -1))
        C = torch.empty_like(R)
        getattr(K, fn)(R, C)
        return host(C).ravel().tolist()

    assert smx("softmax_q19", [0, -(1 << 19)]) == [383193, 141094]
    assert smx("softmax_q19", [0, 0, 0, 0, -(1 << 42), -(1 << 42), -(1 << 42), -(1 << 42)]) == [1 << 17] * 4 + [0] * 4
    assert smx("softmax_q21", [0, -11356, -2924304]) == [933750, 931225, 232177]     # rounded exponent, rounded quotient
    assert smx("softmax_q21", [0, -(1 << 42)]) == [1 << 21, 0]
    assert smx("softmax_q21", [0, -6096986655889]) == [1 << 21, 0]                   # the product wraps: the clip decides
    assert act("sigmoid_q23", [-(1 << 23), 3, -22713, 0]) == [2257517, 4199982, 1 << 22, 1 << 22]
    assert act("silu_q23", [-(1 << 23), -22713, 0]) == [-2257517, -11357, 0]
    assert act("sigmoid_q25", [-90852, 181705, 3, -407108648]) == [16754503, 16822642, 16799929, 180]
    assert act("silu_q25", [-90852, 181705]) == [-45365, 91098]
    # the same values in the middle of a long tensor, where the table kernels and the vector loads take them
    vals = np.zeros(70000, np.int64)
    vals[[5, 4099, 65537]] = [-90852, 181705, -407108648]
    out = np.array(act("sigmoid_q25", vals))
    assert out[[5, 4099, 65537]].tolist() == [16754503, 16822642, 180] and (np.delete(out, [5, 4099, 65537]) == 1 << 24).all()
    vals[[5, 4099, 65537]] = [-22713, -(1 << 23), 3]
    out = np.array(act("sigmoid_q23", vals))
    assert out[[5, 4099, 65537]].tolist() == [1 << 22, 2257517, 4199982]
    row = np.full(1024, -(1 << 42), np.int64)
    row[[0, 500, 1023]] = [0, -11356, -2924304]
    assert np.array(smx("softmax_q21", row))[[0, 500, 1023]].tolist() == [933750, 931225, 232177]


def test_softmax_unaligned_rows(K, oracle):
    rng = np.random.default_rng(3)
    x = _scores(rng, (1, 2, 3, 1024), 19)
    buf = torch.zeros(x.size + 1, dtype=torch.int64, device="cuda")
    R = buf[1:].view(1, 2, 3, 1024)                 # 8-byte aligned only
    R.copy_(dev(x))
    C = torch.empty_like(dev(x))
    K.softmax_q19(R, C)
    assert np.array_equal(host(C), oracle.softmax_q19(x)[0])


def test_softmax_config3_full_size_properties(K, oracle):
    """Benchmark config 3 softmax at full size [1,1024,128,1024]: exact on a sample of rows, invariants on all."""
    g = torch.Generator(device="cpu").manual_seed(3000)
    S, H, T = 1024, 128, 1024
    x = torch.randint(-(6 << 19), 6 << 19, (1, S, H, T), generator=g, dtype=torch.int64)
    mask = torch.full((S, T), -(64 << 36), dtype=torch.int64).triu_(1)
    x += mask.unsqueeze(1)
    R = x.cuda()
    C = torch.empty_like(R)
    K.softmax_q19(R, C)
    assert torch.equal(R.cpu(), x)
    sel = [0, 1, 17, 511, 1023]
    Ce, _ = oracle.softmax_q19(x[:, sel].numpy())
    assert np.array_equal(host(C[:, sel]), Ce)
    assert int(C.min()) >= 0 and int(C.max()) <= 1 << 19
    sums = C.sum(-1)
    assert int(sums.max()) <= 1 << 19 and int(sums.min()) > (1 << 19) - T
    causal = torch.ones((S, T), dtype=torch.bool, device="cuda").triu_(1)
    assert int((C * causal.unsqueeze(1)).abs().max()) == 0            # masked positions get exactly 0


# -------------------------------------------------------------------------------- SiLU / sigmoid --
ACTS = [("silu_q23", 23), ("sigmoid_q23", 23), ("silu_q25", 25), ("sigmoid_q25", 25)]


@pytest.mark.parametrize("fn,Q", ACTS)
@pytest.mark.parametrize("shape", [(1, 1, 1), (1, 3, 7), (2, 5, 256), (1, 128, 2048), (1, 7, 2049)])
def test_activation_shapes(K, oracle, fn, Q, shape):
    rng = np.random.default_rng(Q + sum(shape))
    x = rng.integers(-(20 << Q), 20 << Q, size=shape, dtype=np.int64)
    R = dev(x)
    C = torch.empty_like(R)
    getattr(K, fn)(R, C)
    assert np.array_equal(host(C), getattr(oracle, fn)(x))
    assert np.array_equal(host(R), x)


@pytest.mark.parametrize("fn,Q", ACTS)
def test_activation_edges_and_hazard_region(K, oracle, fn, Q):
    """saturation limits, zero, the overflowing-shift region x <= -27.7 (k >= 40), full-range garbage and a
    hostile table: everything must match the oracle's fixed semantics bit for bit"""
    one = 1 << Q
    rng = np.random.default_rng(Q)
    edges = np.array([0, 1, -1, 64 * one, 64 * one - 1, -64 * one, -64 * one + 1, 100 * one, -100 * one,
                      -(1 << 63), (1 << 63) - 1, -28 * one, -44 * one, -45 * one, -63 * one], np.int64)
    x = np.concatenate([edges, rng.integers(-64 * one, -27 * one, size=3000, dtype=np.int64),
                        rand_i64(rng, (3000,), 63)]).reshape(1, 1, -1)
    lut_bad = rand_i64(rng, (256,), 63)
    default = K.EXP2_FRAC_LUT_Q23 if Q == 23 else K.EXP2_FRAC_LUT_Q25
    for table in (None, lut_bad):
        R = dev(x)
        C = torch.empty_like(R)
        t = default if table is None else dev(table)
        getattr(K.lib, fn)(R.data_ptr(), C.data_ptr(), t.data_ptr(), 1, 1, x.shape[2])
        torch.cuda.synchronize()
        assert np.array_equal(host(C), getattr(oracle, fn)(x, table))


def test_activation_unaligned_pointers(K, oracle):
    rng = np.random.default_rng(8)
    x = rng.integers(-(20 << 23), 20 << 23, size=(1, 3, 1001), dtype=np.int64)
    buf = torch.zeros(x.size + 1, dtype=torch.int64, device="cuda")
    R = buf[1:].view(1, 3, 1001)
    R.copy_(dev(x))
    C = torch.empty_like(dev(x))
    K.silu_q23(R, C)
    assert np.array_equal(host(C), oracle.silu_q23(x))


def test_activation_dense_ffn_shape(K, oracle):
    """[1,512,18432], the dense-FFN activation shape; oracle on everything (9.4 M elements)."""
    g = torch.Generator(device="cpu").manual_seed(2300)
    x = torch.randint(-(16 << 23), 16 << 23, (1, 512, 18432), generator=g, dtype=torch.int64)
    R = x.cuda()
    C = torch.empty_like(R)
    oracle.set_threads(oracle.max_threads())
    for fn in ("silu_q23", "sigmoid_q23"):
        getattr(K, fn)(R, C)
        assert np.array_equal(host(C), getattr(oracle, fn)(x.numpy()))
    oracle.set_threads(1)


# ---------------------------------------------------------------------------------- RMSNorm -----
@pytest.mark.parametrize("bits", [20, 37, 63])
@pytest.mark.parametrize("N", [7, 512, 1536, 7168, 9001])
@pytest.mark.parametrize("w32", [True, False])
def test_rmsnorm(K, oracle, bits, N, w32):
    rng = np.random.default_rng(bits + N)
    M = 6
    A = rand_i64(rng, (M, N), bits)
    if bits == 63:
        A[0, :] = (1 << 63) - 1
    W = rng.integers(1 << 5, 1 << 20, size=(N,), dtype=np.int32) if w32 else rand_i64(rng, (N,), 40)
    C, rms = K.RMS_Norm_int64(dev(A), dev(W), 1, N)
    Ce, rmse = oracle.RMS_Norm_int64(A, W, 1, N)
    assert rms.shape == (500,) and rms.device.type == "cpu"
    assert np.array_equal(rms[:M].numpy(), rmse)
    assert np.array_equal(host(C), Ce)


def test_rmsnorm_reference_entry_points(K, oracle):
    """rms_norm_32 / rms_norm_64 with a caller-supplied rms vector (the reference's contract), including
    negative and huge divisors that only the slow exact path handles"""
    rng = np.random.default_rng(12)
    A = rand_i64(rng, (5, 300), 63)
    rms = np.array([1, -3, 12345678901, (1 << 62) + 12345, 977], np.int64)
    for W in (rand_i32(rng, (300,)), rand_i64(rng, (300,), 63)):
        C = torch.empty((5, 300), dtype=torch.int64, device="cuda")
        fn = K.lib.rms_norm_32 if W.dtype == np.int32 else K.lib.rms_norm_64
        Ad, Wd, rd = dev(A), dev(W), dev(rms)
        fn(Ad.data_ptr(), Wd.data_ptr(), rd.data_ptr(), C.data_ptr(), 5, 300)
        torch.cuda.synchronize()
        assert np.array_equal(host(C), oracle.rms_norm_apply(A, W, rms))
    assert K.int64_RMS0(dev(A[0]), 1, 300) == int(oracle.rms_stat(A[:1], 1, 300)[0])


@pytest.mark.parametrize("bits", [12, 40, 56])       # (the sums stay below 2^126: 977 squares of 55 bits)
def test_rms_statistic_divisors(K, oracle, bits):
    """the statistic's 192-bit division takes a different route below 2^20, below 2^32 and beyond: divisors on both
    sides of each border, and sums whose quotient digits sit next to a multiple of the divisor"""
    rng = np.random.default_rng(bits)
    rows = [rand_i64(rng, (977,), bits), np.full(977, (1 << (bits - 1)) - 1, np.int64), np.zeros(977, np.int64)]
    rows[2][:3] = [1 << (bits // 2), 3, -1]
    for dim in (1, 2, 7, 977, 7168, (1 << 20) - 1, 1 << 20, (1 << 20) + 1, (1 << 32) - 1, 1 << 32, (1 << 40) + 9):
        for eps in (1, dim - 1, dim, (1 << 31) + 5):
            if eps < 1:
                continue
            for a in rows:
                assert K.int64_RMS0(dev(a), eps, dim) == int(oracle.rms_stat(a[None], eps, dim)[0]), (dim, eps)


@pytest.mark.parametrize("w32", [True, False])
@pytest.mark.parametrize("r", [3, 977, (1 << 31) - 1, (1 << 36) + 12345, (1 << 52) + 3, (1 << 61) + 5])
def test_rmsnorm_quotients_next_to_integers(K, oracle, r, w32):
    """a * w / r exactly on, one below and one above multiples of r, at quotients from 0 to beyond 2^49, both signs:
    the cases a floating-point estimate of the quotient cannot settle and the exact tiers behind it must"""
    rng = np.random.default_rng(r % 1000)
    N = 1024
    n = np.concatenate([np.arange(-8, 8), rng.integers(-(1 << 20), 1 << 20, 200), rng.integers(-(1 << 40), 1 << 40, 200),
                        rng.integers(-(1 << 51), 1 << 51, 100), [(1 << 49) - 1, 1 << 49, -(1 << 49), (1 << 50) + 1]])
    prods = []
    for q in n.tolist():
        for delta in (-1, 0, 1, r - 1, -(r - 1), r // 2):
            p = q * r + delta
            if -(1 << 63) <= p < (1 << 63):
                prods.append(p)
    prods = np.array(prods[: (len(prods) // N) * N], dtype=np.int64).reshape(-1, N)
    M = prods.shape[0]
    # w = 1: the product is a itself; w = -1 and a small factor exercise the sign and a genuine multiplication
    for wv, A in ((1, prods), (-1, -np.maximum(prods, -(1 << 63) + 1)), (3, prods // 3)):
        W = np.full((N,), wv, dtype=np.int32 if w32 else np.int64)
        rms = np.full((M,), r, dtype=np.int64)
        C = torch.empty((M, N), dtype=torch.int64, device="cuda")
        fn = K.lib.rms_norm_32 if w32 else K.lib.rms_norm_64
        Ad, Wd, rd = dev(A), dev(W), dev(rms)
        fn(Ad.data_ptr(), Wd.data_ptr(), rd.data_ptr(), C.data_ptr(), M, N)
        torch.cuda.synchronize()
        K._check("rms_norm")
        assert np.array_equal(host(C), oracle.rms_norm_apply(np.ascontiguousarray(A), W, rms))


@pytest.mark.parametrize("N", [7, 512, 1536, 4096, 7168, 9001, 20000])
@pytest.mark.parametrize("k,w32,inplace", [(12, True, False), (8, False, True), (0, True, True), (63, False, False)])
def test_rmsnorm_residual_fusion(K, oracle, N, k, w32, inplace):
    """x + y * 2^k (wrapping) stored and normalised in one pass (model.py:1465-1468): every row-length tier, odd and
    even N, in place or not, sums that wrap around 2^64"""
    rng = np.random.default_rng(N + k)
    M = 5
    X = rand_i64(rng, (M, N), 37)
    Y = rand_i64(rng, (M, N), 40 if k < 20 else 63)
    if k == 8:
        X[1, :5] = [(1 << 63) - 1, -(1 << 63), (1 << 62), -1, 0]          # the sum wraps
        Y[1, :5] = [(1 << 54), -(1 << 54) - 1, (1 << 55) - 1, 1, 0]
    W = rng.integers(1 << 5, 1 << 20, size=(N,), dtype=np.int32) if w32 else rand_i64(rng, (N,), 40)
    Xd = dev(X)
    Xn, C, rms = K.RMS_Norm_residual_int64(Xd, dev(Y), k, dev(W), 1, N, inplace=inplace)
    Xe, Ce, rmse = oracle.RMS_Norm_residual_int64(X, Y, k, W, 1, N)
    assert (Xn.data_ptr() == Xd.data_ptr()) == inplace
    assert np.array_equal(host(Xn), Xe)
    assert np.array_equal(rms[:M].numpy(), rmse)
    assert np.array_equal(host(C), Ce)


def test_rmsnorm_residual_fusion_unaligned_and_bad_arguments(K, oracle):
    rng = np.random.default_rng(77)
    M, N = 3, 1000
    X, Y = rand_i64(rng, (M, N), 37), rand_i64(rng, (M, N), 30)
    W = rng.integers(1, 1 << 20, size=(N,), dtype=np.int32)
    # rows that start 8 bytes off a 16-byte boundary take the element-wise path
    buf = torch.zeros((M * N + 1,), dtype=torch.int64, device="cuda")
    Xd = buf[1:].view(M, N)
    Xd.copy_(dev(X))
    Yd, Wd = dev(Y), dev(W)
    Xo = torch.empty((M, N), dtype=torch.int64, device="cuda")
    C = torch.empty((M, N), dtype=torch.int64, device="cuda")
    r = torch.empty((M,), dtype=torch.int64, device="cuda")
    K.lib.rms_norm_residual_fused_32(Xd.data_ptr(), Yd.data_ptr(), 12, Wd.data_ptr(), Xo.data_ptr(), r.data_ptr(), C.data_ptr(), M, N, 1, N)
    torch.cuda.synchronize()
    K._check("residual norm")
    Xe, Ce, rmse = oracle.RMS_Norm_residual_int64(X, Y, 12, W, 1, N)
    assert np.array_equal(host(Xo), Xe) and np.array_equal(host(C), Ce) and np.array_equal(host(r), rmse)
    for bad_k in (-1, 64):
        K.lib.rms_norm_residual_fused_32(Xd.data_ptr(), Yd.data_ptr(), bad_k, Wd.data_ptr(), Xo.data_ptr(), r.data_ptr(), C.data_ptr(), M, N, 1, N)
        assert K.lib.zk_last_error() == 1
        K.lib.zk_clear_error()
    K.lib.rms_norm_residual_fused_32(Xd.data_ptr(), None, 12, Wd.data_ptr(), Xo.data_ptr(), r.data_ptr(), C.data_ptr(), M, N, 1, N)
    assert K.lib.zk_last_error() == 1
    K.lib.zk_clear_error()


def test_rmsnorm_model_shape(K, oracle):
    """[256,7168] at residual-stream magnitudes (|x| up to ~2^37, Q31) with int32 Q21 weights"""
    g = torch.Generator(device="cpu").manual_seed(600)
    A = torch.randint(-(1 << 37), 1 << 37, (256, 7168), generator=g, dtype=torch.int64)
    W = torch.randint(1 << 18, 1 << 20, (7168,), generator=g, dtype=torch.int32)
    C, rms = K.RMS_Norm_int64(A.cuda(), W.cuda(), 1, 7168)
    Ce, rmse = oracle.RMS_Norm_int64(A.numpy(), W.numpy(), 1, 7168)
    assert np.array_equal(rms[:256].numpy(), rmse) and np.array_equal(host(C), Ce)


# ------------------------------------------------------------------------------------- RoPE -----
@pytest.mark.parametrize("bits", [31, 63])
def test_rope(K, oracle, bits):
    rng = np.random.default_rng(bits)
    A = rand_i64(rng, (2, 7, 5, 32, 2), bits)
    Bt = rand_i64(rng, (1, 7, 1, 32, 2), 43)
    out = K.complex_int64_mul_broadcast(dev(A), dev(Bt))
    assert np.array_equal(host(out), oracle.complex_int64_mul_broadcast(A, Bt))


def test_gemm_mfma_path_is_taken(K, oracle):
    """the i8 MFMA path must really run (and report its digit counts) on the shapes it is meant for"""
    rng = np.random.default_rng(42)
    A = rand_i64(rng, (1, 64, 256), 20)
    W = rand_i64(rng, (128, 256), 16)
    K.lib.zk_gemm_set_path(2)
    dA, dW = dev(A), dev(W)
    Ce, Re = oracle.int64_bmm_broadcast(A, W, 1, 1, 29)
    for _ in range(3):          # (a first call may run on digits remembered for other operands at these addresses)
        C, R = K.int64_bmm_broadcast(dA, dW, 1, 1, 29)
        assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
    assert K.gemm_last_plan() == (2, 3, 3)
    A = rand_i64(rng, (1, 64, 256), 63)
    W = rand_i64(rng, (128, 256), 63)
    dA2, dW2 = dev(A), dev(W)            # the first pair stays alive: new addresses, nothing remembered about them
    # (operands at new addresses run on the digits of the last operands of their shape, here the pair above: the
    # guarded launch behind the product redoes it, and what the kernels saw reaches the next call)
    hits = K.lib.zk_gemm_guard_hits()
    C, R = K.int64_bmm_broadcast(dA2, dW2, 1, 1, 29)
    Ce, Re = oracle.int64_bmm_broadcast(A, W, 1, 1, 29)
    assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
    # (no recomputation only if the allocator handed out addresses last seen with nine-digit operands)
    assert K.lib.zk_gemm_guard_hits() in (hits, hits + 1)
    C, R = K.int64_bmm_broadcast(dA2, dW2, 1, 1, 29)
    assert K.gemm_last_plan() == (2, 9, 9)
    assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
    K.lib.zk_gemm_set_path(1)
    C, R = K.int64_bmm_broadcast(dA2, dW2, 1, 1, 29)
    assert K.gemm_last_plan() == (1, 0, 0)
    K.lib.zk_gemm_set_path(0)


@pytest.mark.parametrize("M", [20, 48])
def test_gemm_stale_digit_guess_is_caught(K, oracle, M):
    """Operands that change in place under the same pointers.  The call after the change runs on the digit
    counts remembered for those pointers and does not wait for their check; the guarded recomputation behind
    it must still deliver exact results, and the following call must have learnt the new range."""
    rng = np.random.default_rng(7 + M)
    A = rand_i64(rng, (1, M, 512), 20)
    W = rand_i64(rng, (160, 512), 16)
    dA, dW = dev(A), dev(W)
    K.lib.zk_gemm_set_path(2)
    # (torch may hand out addresses an earlier test used with wider operands: the first call then still runs on the
    # digit counts remembered for them, and the range it reports corrects that for the next one)
    for _ in range(3):
        C, R = K.int64_bmm_broadcast(dA, dW, 1, 1, 29)
        torch.cuda.synchronize()
    assert K.gemm_last_plan() == (2, 3, 3)
    Ce, Re = oracle.int64_bmm_broadcast(A, W, 1, 1, 29)
    assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
    hits = K.lib.zk_gemm_guard_hits()

    A2 = rand_i64(rng, A.shape, 63)
    W2 = rand_i64(rng, W.shape, 40)
    dA.copy_(torch.from_numpy(A2))
    dW.copy_(torch.from_numpy(W2))
    C, R = K.int64_bmm_broadcast(dA, dW, 1, 1, 29)
    assert K.gemm_last_plan() == (2, 3, 3), "this call is expected to run on the stale guess"
    Ce, Re = oracle.int64_bmm_broadcast(A2, W2, 1, 1, 29)
    assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
    assert K.lib.zk_gemm_guard_hits() == hits + 1
    C, R = K.int64_bmm_broadcast(dA, dW, 1, 1, 29)
    assert K.gemm_last_plan()[0] == 2 and K.gemm_last_plan()[1] == 9 and K.gemm_last_plan()[2] >= 6
    assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
    assert K.lib.zk_gemm_guard_hits() == hits + 1

    # and back: one call on digit counts that are wider than needed, then the narrow ones again
    dA.copy_(torch.from_numpy(A))
    dW.copy_(torch.from_numpy(W))
    Ce, Re = oracle.int64_bmm_broadcast(A, W, 1, 1, 29)
    C, R = K.int64_bmm_broadcast(dA, dW, 1, 1, 29)
    assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
    C, R = K.int64_bmm_broadcast(dA, dW, 1, 1, 29)
    assert K.gemm_last_plan() == (2, 3, 3)
    assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
    K.lib.zk_gemm_set_path(0)


@pytest.mark.parametrize("fn,Q", ACTS)
def test_activation_table_path(K, oracle, fn, Q):
    """tensors of 2^20 elements or more take the quotient-table kernel: in-range values, both saturation sides, the
    shifts outside the table (|x| > 16.6), the overflowing-shift region, full-range garbage and a hostile table (which
    must switch the kernel back to per-element division) all have to match the oracle"""
    one = 1 << Q
    rng = np.random.default_rng(100 + Q)
    n = (1 << 20) + 3
    x = rng.integers(-(18 << Q), 18 << Q, size=n, dtype=np.int64)
    x[:4000] = rng.integers(-64 * one, 64 * one, size=4000, dtype=np.int64)
    x[4000:8000] = rand_i64(rng, (4000,), 63)
    x[8000:8016] = [0, 1, -1, 64 * one, 64 * one - 1, -64 * one, -64 * one + 1, 100 * one, -100 * one, -(1 << 63),
                    (1 << 63) - 1, -28 * one, -44 * one, -45 * one, -63 * one, 17 * one]
    x = x.reshape(1, 1, n)
    oracle.set_threads(oracle.max_threads())
    default = K.EXP2_FRAC_LUT_Q23 if Q == 23 else K.EXP2_FRAC_LUT_Q25
    for table in (None, rand_i64(rng, (256,), 63), rng.integers(0, 1 << 40, size=256, dtype=np.int64)):
        R = dev(x)
        C = torch.empty_like(R)
        t = default if table is None else dev(table)
        getattr(K.lib, fn)(R.data_ptr(), C.data_ptr(), t.data_ptr(), 1, 1, n)
        torch.cuda.synchronize()
        K._check(fn)
        assert np.array_equal(host(C), getattr(oracle, fn)(x, table))
    oracle.set_threads(1)


@pytest.mark.parametrize("fn,Q", ACTS)
def test_activation_quotients_follow_the_table(K, oracle, fn, Q):
    """the quotients made from the caller's table are kept between calls: a table rewritten in place under the same
    pointer, and the old table coming back, must show in the very next call and in the calls after it, whether or not
    the host has waited for the device in between"""
    rng = np.random.default_rng(300 + Q)
    n = (1 << 20) + 2
    x = rng.integers(-(18 << Q), 18 << Q, size=(1, 1, n), dtype=np.int64)
    default = host(K.EXP2_FRAC_LUT_Q23 if Q == 23 else K.EXP2_FRAC_LUT_Q25)
    tables = [default, rng.integers(0, 1 << 40, size=256, dtype=np.int64), default,
              default + rng.integers(0, 2, size=256, dtype=np.int64), rand_i64(rng, (256,), 63)]
    oracle.set_threads(oracle.max_threads())
    R = dev(x)
    t = dev(default.copy())
    for i, table in enumerate(tables):
        t.copy_(torch.from_numpy(table))                  # in place: the pointer stays the same
        expect = getattr(oracle, fn)(x, table)
        outs = []
        for rep in range(4):
            C = torch.empty_like(R)
            getattr(K.lib, fn)(R.data_ptr(), C.data_ptr(), t.data_ptr(), 1, 1, n)
            if (rep + i) & 1:
                torch.cuda.synchronize()
            outs.append(C)
        torch.cuda.synchronize()
        K._check(fn)
        for rep, C in enumerate(outs):
            assert np.array_equal(host(C), expect), "table %d, call %d" % (i, rep)
    oracle.set_threads(1)


@pytest.mark.parametrize("T", [1, 7, 64, 100, 1024, 2048, 2050, 3001])
@pytest.mark.parametrize("with_s2,with_mask,keep_scores", [(True, True, True), (False, False, False), (True, False, True), (False, True, False)])
def test_softmax_q19_scores_fusion(K, oracle, T, with_s2, with_mask, keep_scores):
    """fused score preparation + softmax against the op-by-op restatement (inference/model.py:896-915)"""
    if T > 2048 and not keep_scores:
        pytest.skip("rows longer than 2048 need the scores buffer")
    rng = np.random.default_rng(T * 8 + with_s2 * 4 + with_mask * 2 + keep_scores)
    shape = (2, 3, 5, T)
    s1 = rng.integers(-(40 << 19), 40 << 19, size=shape, dtype=np.int64)
    s2 = rng.integers(-(40 << 19), 40 << 19, size=shape, dtype=np.int64) if with_s2 else None
    s1.ravel()[:3] = [(1 << 62) + 12345, -(1 << 62) - 999, -1]        # the multiplication by 94 wraps, as in torch
    mask = np.triu(np.full((3, T), -(64 << 36), np.int64), 1) if with_mask else None
    C = torch.empty(shape, dtype=torch.int64, device="cuda")
    scores = torch.empty(shape, dtype=torch.int64, device="cuda") if keep_scores else None
    K.softmax_q19_scores(dev(s1), None if s2 is None else dev(s2), None if mask is None else dev(mask), C, scores)
    xe, Ce = oracle.softmax_q19_scores(s1, s2, mask)
    if keep_scores:
        assert np.array_equal(host(scores), xe)
    assert np.array_equal(host(C), Ce)


def test_softmax_q19_scores_other_divisors_and_alignment(K, oracle):
    rng = np.random.default_rng(5)
    shape = (1, 4, 2, 129)
    s1 = rng.integers(-(1 << 40), 1 << 40, size=shape, dtype=np.int64)
    s2 = rng.integers(-(1 << 40), 1 << 40, size=shape, dtype=np.int64)
    for mul, div in ((1, 1), (-3, 7), (94, 695), (12345, (1 << 31) - 1)):
        C = torch.empty(shape, dtype=torch.int64, device="cuda")
        sc = torch.empty(shape, dtype=torch.int64, device="cuda")
        K.softmax_q19_scores(dev(s1), dev(s2), None, C, sc, mul=mul, div=div)
        xe, Ce = oracle.softmax_q19_scores(s1, s2, None, mul, div)
        assert np.array_equal(host(sc), xe), (mul, div)
        assert np.array_equal(host(C), Ce), (mul, div)
    with pytest.raises(RuntimeError):
        K.softmax_q19_scores(dev(s1), dev(s2), None, C, sc, div=0)
    K.lib.zk_clear_error()


@pytest.mark.parametrize("shape", [(1, 1, 1), (1, 3, 7), (2, 5, 129), (1, 64, 2048), (1, 600, 2048)])
@pytest.mark.parametrize("keep", [False, True])
def test_silu_mul_q23_fusion(K, oracle, shape, keep):
    """fused SiLU gate product against silu_q23 followed by the reference's tensor ops (inference/model.py:1039-1048);
    the largest shape takes the quotient-table kernel"""
    rng = np.random.default_rng(sum(shape) + keep)
    r = rng.integers(-(20 << 23), 20 << 23, size=shape, dtype=np.int64)
    u = rng.integers(-(1 << 45), 1 << 45, size=shape, dtype=np.int64)
    r.ravel()[0] = 70 << 23                                          # the pass-through branch: silu(x) = x
    C = torch.empty(shape, dtype=torch.int64, device="cuda")
    S = torch.empty(shape, dtype=torch.int64, device="cuda") if keep else None
    K.silu_mul_q23(dev(r), dev(u), C, S)
    se, ce = oracle.silu_mul_q23(r, u)
    assert np.array_equal(host(C), ce)
    if keep:
        assert np.array_equal(host(S), se)


# (the shapes with 2..16 groups of 8, 16 or 32 experts run on the lane-per-group kernel, the others on the wave-wide one;
#  (64, 8, 2, 40) and (32, 2, 1, 20) ask for more winners than the kept groups hold, so masked experts win too)
GATE_SHAPES = [(256, 8, 4, 8), (16, 4, 2, 4), (64, 1, 1, 6), (96, 3, 3, 5), (512, 8, 3, 8), (1024, 16, 5, 64), (7, 1, 1, 7),
               (512, 16, 4, 6), (64, 4, 2, 9), (64, 8, 2, 40), (32, 2, 1, 20), (128, 16, 16, 64), (64, 2, 2, 3)]


@pytest.mark.parametrize("E,G,KG,K_", GATE_SHAPES)
@pytest.mark.parametrize("with_bias", [True, False])
def test_gate_route(K, oracle, E, G, KG, K_, with_bias):
    """routing of Gate.forward on the device against the oracle, ties included (coarse scores tie often)"""
    rng = np.random.default_rng(E * 3 + G + with_bias)
    # (beyond 8192 tokens the lane-per-group kernel switches from four lanes per group to one)
    for T, hi in ((1, 1 << 23), (77, 1 << 23), (300, 12), (1031, 1 << 23), (8200, 1 << 23), (8195, 9)):
        scores = rng.integers(1, hi, size=(T, E), dtype=np.int64)
        bias = rng.integers(-(hi >> 3) - 1, (hi >> 3) + 1, size=E, dtype=np.int64).astype(np.int32) if with_bias else None
        raw = torch.empty((T, K_), dtype=torch.int64, device="cuda")
        w, idx = K.gate_route(dev(scores), None if bias is None else dev(bias), G, KG, K_, raw)
        we, ie, re_ = oracle.gate_route(scores, bias, G, KG, K_)
        assert np.array_equal(host(idx), ie), "indices"
        assert np.array_equal(host(raw), re_), "gathered scores"
        assert np.array_equal(host(w), we), "weights"


@pytest.mark.parametrize("E,G,KG,K_", GATE_SHAPES)
@pytest.mark.parametrize("with_bias", [True, False])
def test_gate_sigmoid_route(K, oracle, E, G, KG, K_, with_bias):
    """sigmoid and routing in one launch against the oracle's sigmoid_q23 followed by its routing: logits over the
    sigmoid's whole domain (the ends saturate, so scores tie), with and without the scores written"""
    rng = np.random.default_rng(E * 5 + G + with_bias)
    for T, span in ((1, 1 << 26), (130, 1 << 24), (515, 1 << 31), (64, 40), (8197, 1 << 25)):
        logits = rng.integers(-span, span, size=(T, E), dtype=np.int64)
        bias = rng.integers(-(1 << 20), 1 << 20, size=E, dtype=np.int64).astype(np.int32) if with_bias else None
        sig = oracle.sigmoid_q23(logits[None])[0]
        we, ie, re_ = oracle.gate_route(sig, bias, G, KG, K_)
        for keep in (True, False):
            raw = torch.empty((T, K_), dtype=torch.int64, device="cuda")
            sc, w, idx = K.gate_sigmoid_route(dev(logits), None if bias is None else dev(bias), G, KG, K_, raw, keep_scores=keep)
            assert (sc is None) == (not keep)
            if keep:
                assert np.array_equal(host(sc), sig), "sigmoid scores"
            assert np.array_equal(host(idx), ie), "indices"
            assert np.array_equal(host(raw), re_), "gathered scores"
            assert np.array_equal(host(w), we), "weights"


def _routing(rng, T, E, Kr):
    """Kr distinct experts per token; some experts deliberately left without tokens"""
    live = rng.permutation(E)[: max(Kr, (E * 3) // 4)]
    return np.stack([rng.permutation(live)[:Kr] for _ in range(T)]).astype(np.int64)


@pytest.mark.parametrize("T,E,Kr", [(1, 8, 2), (5, 4, 4), (100, 16, 3), (256, 256, 8), (700, 32, 6), (300, 700, 4), (2000, 257, 1)])
def test_moe_dispatch(K, oracle, T, E, Kr):
    rng = np.random.default_rng(T + E)
    idx = _routing(rng, T, E, Kr)
    d = K.moe_dispatch(dev(idx), E)
    seg, tok, pos = oracle.moe_dispatch(idx, E)
    assert np.array_equal(host(d["seg"]), seg)
    assert np.array_equal(host(d["token"]), tok)
    assert np.array_equal(host(d["pos"]), pos)
    nt = int(host(d["ntiles"])[0])
    tiles = host(d["tiles"])[: 2 * nt].reshape(nt, 2)
    want = [(e, r) for e in range(E) for r in range(int(seg[e]), int(seg[e + 1]), 32)]
    assert tiles.tolist() == [list(t) for t in want]


def test_moe_dispatch_reports_indices_outside_the_experts(K, oracle, monkeypatch):
    """an expert index outside [0, E) belongs to no segment: nothing may read outside the buffers (the entry points at
    row 0, the unowned rows get token 0), the valid entries are placed as ever, and the error channel reports the call"""
    rng = np.random.default_rng(5)
    T, E, Kr, N = 50, 16, 4, 64
    idx = _routing(rng, T, E, Kr)
    bad = [(3, 1, -1), (20, 0, E), (49, 3, 1 << 40)]
    for t, k, v in bad:
        idx[t, k] = v
    # (the kernels report through a flag in host memory: the wrapper's own check raises if they were quick enough, so
    #  it is held off here and the error is read once the stream has drained)
    with monkeypatch.context() as mp:
        mp.setattr(K, "_check", lambda what: None)
        d = K.moe_dispatch(dev(idx), E)
    torch.cuda.synchronize()
    assert K.lib.zk_last_error() == 1 and b"outside" in K.lib.zk_last_error_string()
    K.lib.zk_clear_error()
    valid = (idx >= 0) & (idx < E)
    seg, tok, pos = oracle.moe_dispatch(np.where(valid, idx, E), E + 1)      # the invalid ones sorted behind everything else
    rows = T * Kr - len(bad)
    assert np.array_equal(host(d["seg"]), seg[: E + 1]) and int(seg[E]) == rows
    assert np.array_equal(host(d["token"])[:rows], tok[:rows]) and not host(d["token"])[rows:].any()
    assert np.array_equal(host(d["pos"])[valid], pos[valid]) and not host(d["pos"])[~valid].any()
    # the steps behind it run on what the dispatch left, inside their buffers
    x = rand_i64(rng, (T, N), 30)
    xs = K.moe_gather_rows(dev(x), d)
    assert np.array_equal(host(xs)[:rows], x[tok[:rows]]) and np.array_equal(host(xs)[rows:], np.broadcast_to(x[0], (len(bad), N)))
    w = rand_i64(rng, (T, Kr), 23)
    y = K.moe_combine(xs, dev(w), d, T)
    p = np.where(valid, pos, 0)
    ye = np.zeros((T, N), dtype=np.int64)
    for k in range(Kr):
        ye += (host(xs)[p[:, k]] * w[:, k:k + 1]) >> 23
    assert np.array_equal(host(y), ye)


@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("w32", [False, True])
@pytest.mark.parametrize("bits", [(20, 16), (37, 30), (50, 31)])
def test_int64_grouped_bmm(K, oracle, path, w32, bits):
    """one launch over all experts against the per-expert oracle GEMMs: empty experts, experts with more than 32
    rows, ragged K and N, the remainder output; (50, 31)-bit operands are wider than five digits, which the wavefronts
    that meet them recompute on the vector ALU"""
    rng = np.random.default_rng(bits[0] + w32)
    T, E, Kr, Kd, N = 90, 12, 3, 200, 300
    idx = _routing(rng, T, E, Kr)
    idx[:60, 0] = 2                                           # expert 2 gets more than 32 rows
    idx[:60, 1:] = np.stack([rng.permutation([0, 1, 3, 4, 5])[: Kr - 1] for _ in range(60)])
    x = rand_i64(rng, (T, Kd), bits[0])
    ws = [rand_i32(rng, (N, Kd), bits[1]) if w32 else rand_i64(rng, (N, Kd), bits[1]) for _ in range(E)]
    K.lib.zk_gemm_set_path(path)
    d = K.moe_dispatch(dev(idx), E)
    xs = K.moe_gather_rows(dev(x), d)
    seg, tok, _ = oracle.moe_dispatch(idx, E)
    assert np.array_equal(host(xs), x[tok])
    wd = [dev(w) for w in ws]
    before = K.lib.zk_gemm_grouped_mfma_calls()
    for c in (0, 19):
        C, R = K.int64_grouped_bmm(xs, K.pointer_table(wd), w32, N, c, d, want_remainder=True)
        Ce, Re = oracle.grouped_bmm(x[tok], ws, seg, c)
        assert np.array_equal(host(C), Ce), "quotient"
        assert np.array_equal(host(R), Re), "remainder"
    assert K.lib.zk_gemm_grouped_mfma_calls() - before == (2 if path != 1 else 0), "which route the product took"
    K.lib.zk_gemm_set_path(0)


@pytest.mark.parametrize("w32", [False, True])
@pytest.mark.parametrize("T,Kr,Kd,N", [(1, 8, 520, 300), (2, 8, 7168, 64), (4, 3, 333, 1030), (1, 1, 64, 5000), (8, 8, 520, 300),
                                       (1, 8, 8200, 300), (2, 8, 260, 4200)])
def test_int64_grouped_bmm_few_rows(K, oracle, w32, T, Kr, Kd, N):
    """a decoding step's routed experts: up to 32 rows (64 with int32 weights and K % 4 == 0) go row by row through the
    matrix-vector kernels in one launch (every row against the weights of its own expert, empty experts in between, odd
    K, several staging rounds, the remainder output)"""
    rng = np.random.default_rng(T * 100 + Kr + w32)
    E = 16
    idx = _routing(rng, T, E, Kr)
    x = rand_i64(rng, (T, Kd), 40)
    ws = [rand_i32(rng, (N, Kd), 31) if w32 else rand_i64(rng, (N, Kd), 50) for _ in range(E)]
    K.lib.zk_gemm_set_path(0)
    d = K.moe_dispatch(dev(idx), E)
    xs = K.moe_gather_rows(dev(x), d)
    seg, tok, _ = oracle.moe_dispatch(idx, E)
    wd = [dev(w) for w in ws]
    before = K.lib.zk_gemm_grouped_mfma_calls()
    for c in (0, 23):
        C, R = K.int64_grouped_bmm(xs, K.pointer_table(wd), w32, N, c, d, want_remainder=True)
        Ce, Re = oracle.grouped_bmm(x[tok], ws, seg, c)
        assert np.array_equal(host(C), Ce), "quotient"
        assert np.array_equal(host(R), Re), "remainder"
    if T * Kr <= 32 or w32:
        assert K.lib.zk_gemm_grouped_mfma_calls() == before and K.gemm_last_plan()[0] == 1


@pytest.mark.parametrize("min_pairs", [None, "0"])
@pytest.mark.parametrize("T", [90, 24])
@pytest.mark.parametrize("bits,top,Kd", [((20, 16), False, 224), ((28, 28), False, 224), ((37, 30), False, 96), ((36, 31), True, 224),
                                         ((30, 31), True, 32), ((28, 24), False, 64), ((28, 28), False, 160)])
def test_int64_grouped_bmm_int32_weights_streamed(K, oracle, monkeypatch, min_pairs, T, bits, top, Kd):
    """the grouped launch that streams int32 weights through LDS rings (whole steps of K, sixteen digit pairs or more,
    or any count with ZK_STREAM32_MIN_PAIRS=0): every pair of digit counts it is built for, fewer steps of K than the
    ring has stages, an odd and an even number of steps, experts with no rows, with a few rows (tiles of at most 16 rows
    multiply on v_mfma_i32_16x16x64_i8, two steps at a time) and with more than a tile's 32, a ragged last tile column,
    the remainder output, weights that reach INT32_MAX (a fifth digit); the first call reads its verdict back, the
    later ones run ahead of it behind a guarded launch"""
    if min_pairs is None:
        monkeypatch.delenv("ZK_STREAM32_MIN_PAIRS", raising=False)
    else:
        monkeypatch.setenv("ZK_STREAM32_MIN_PAIRS", min_pairs)
    K.lib.zk_reload_env()
    try:
        rng = np.random.default_rng(bits[0] * 64 + bits[1] + Kd + T)
        E, Kr, N = 12, 3, 300
        idx = _routing(rng, T, E, Kr)
        many = 2 * T // 3
        idx[:many, 0] = 2                                     # expert 2: 60 rows (two tiles), or 16 (the most the 16-row form takes)
        idx[:many, 1:] = np.stack([rng.permutation([0, 1, 3, 4, 5])[: Kr - 1] for _ in range(many)])
        x = rand_i64(rng, (T, Kd), bits[0])
        ws = [rand_i32(rng, (N, Kd), bits[1]) for _ in range(E)]
        if top:
            ws[2][7, 5] = np.iinfo(np.int32).max
            ws[4][299, Kd - 1] = np.iinfo(np.int32).min
        K.lib.zk_gemm_set_path(2)
        d = K.moe_dispatch(dev(idx), E)
        xs = K.moe_gather_rows(dev(x), d)
        seg, tok, _ = oracle.moe_dispatch(idx, E)
        wd = [dev(w) for w in ws]
        table = K.pointer_table(wd)
        for c in (0, 19, 19):
            streamed = K.lib.zk_gemm_grouped_streamed_calls()
            C, R = K.int64_grouped_bmm(xs, table, True, N, c, d, want_remainder=True)
            Ce, Re = oracle.grouped_bmm(x[tok], ws, seg, c)
            assert np.array_equal(host(C), Ce), "quotient"
            assert np.array_equal(host(R), Re), "remainder"
        # (the first calls may run on digit counts that other operands left behind at these addresses; the last does not)
        la, lb = K.gemm_last_plan()[1:]
        assert la <= 5 and lb <= 5
        took = K.lib.zk_gemm_grouped_streamed_calls() - streamed
        assert took == (1 if min_pairs == "0" or la * lb >= 16 else 0), (la, lb, took)
    finally:
        K.lib.zk_gemm_set_path(0)
        monkeypatch.delenv("ZK_STREAM32_MIN_PAIRS", raising=False)
        K.lib.zk_reload_env()


def test_int64_grouped_bmm_int32_weights_streamed_odd_operands(K, oracle, monkeypatch):
    """what the streamed kernel does not take goes another way with the same bits: a K that is no multiple of 32, and one
    expert's matrix at an address that is not a multiple of 16 (the kernel's workgroups for that expert report the full
    range and the product is computed again on other kernels)"""
    monkeypatch.setenv("ZK_STREAM32_MIN_PAIRS", "0")
    K.lib.zk_reload_env()
    try:
        rng = np.random.default_rng(4242)
        T, E, Kr, N = 40, 6, 2, 260
        idx = _routing(rng, T, E, Kr)
        seg, tok, _ = oracle.moe_dispatch(idx, E)
        K.lib.zk_gemm_set_path(0)
        d = K.moe_dispatch(dev(idx), E)
        for Kd, shifted in ((200, False), (128, True)):
            x = rand_i64(rng, (T, Kd), 30)
            ws = [rand_i32(rng, (N, Kd), 27) for _ in range(E)]
            xs = K.moe_gather_rows(dev(x), d)
            wd = [dev(w) for w in ws]
            if shifted:
                flat = torch.zeros(N * Kd + 1, dtype=torch.int32, device="cuda")
                flat[1:] = wd[3].reshape(-1)
                wd[3] = flat[1:].view(N, Kd)
                assert wd[3].data_ptr() % 16 == 4
            table = K.pointer_table(wd)
            streamed = K.lib.zk_gemm_grouped_streamed_calls()
            for c in (0, 17):
                C, R = K.int64_grouped_bmm(xs, table, True, N, c, d, want_remainder=True)
                Ce, Re = oracle.grouped_bmm(x[tok], ws, seg, c)
                assert np.array_equal(host(C), Ce), ("quotient", Kd, shifted, c)
                assert np.array_equal(host(R), Re), ("remainder", Kd, shifted, c)
            if not shifted:
                assert K.lib.zk_gemm_grouped_streamed_calls() == streamed, "K % 32 != 0 is the general kernel's"
    finally:
        monkeypatch.delenv("ZK_STREAM32_MIN_PAIRS", raising=False)
        K.lib.zk_reload_env()


@pytest.mark.parametrize("seed", range(10 * SEEDS))
def test_grouped_bmm_seeded_random_problems(K, oracle, seed):
    """the grouped launch on randomly drawn routings, shapes, operand widths, weight types and shifts: experts without
    rows, with a handful and with several tiles' worth; whole and ragged steps of K (the streamed int32 kernel takes the
    former), ragged tile columns; a few rows in all (the matrix-vector kernels) or many; digits the 32-row kernels
    hold or not (the 16-row kernels behind them); every problem twice, the second call on what the first one learnt"""
    rng = np.random.default_rng(9900 + seed)
    for _ in range(4):
        T = int(rng.choice([1, 3, 8, 40, 150, 400]))
        E = int(rng.choice([2, 8, 16, 40]))
        Kr = int(rng.choice([1, 2, 4]))
        Kr = min(Kr, E)
        Kd = int(rng.choice([32, 64, 96, 160, 200, 224, 520]))
        N = int(rng.choice([16, 64, 250, 256, 300, 700]))
        while T * Kr * Kd * N > 80_000_000:
            T = max(1, T // 2)
        w32 = bool(rng.integers(0, 3))
        bits_a = int(rng.choice([12, 20, 28, 31, 37, 47, 60]))
        bits_w = int(rng.choice([12, 16, 24, 28, 31])) if w32 else int(rng.choice([16, 24, 33, 50]))
        c = int(rng.choice([0, 8, 17, 23, 31, 40]))
        idx = _routing(rng, T, E, Kr)
        if T >= 40 and rng.integers(0, 2):
            idx[: T // 2, 0] = int(idx[0, 0])                # one expert with several tiles
            for t in range(T // 2):
                others = [e for e in rng.permutation(E) if e != idx[t, 0]][: Kr - 1]
                idx[t, 1:] = others
        x = rand_i64(rng, (T, Kd), bits_a)
        ws = [rand_i32(rng, (N, Kd), bits_w) if w32 else rand_i64(rng, (N, Kd), bits_w) for _ in range(E)]
        d = K.moe_dispatch(dev(idx), E)
        xs = K.moe_gather_rows(dev(x), d)
        seg, tok, _ = oracle.moe_dispatch(idx, E)
        wd = [dev(w) for w in ws]
        table = K.pointer_table(wd)
        Ce, Re = oracle.grouped_bmm(x[tok], ws, seg, c)
        for rep in range(2):
            C, R = K.int64_grouped_bmm(xs, table, w32, N, c, d, want_remainder=True)
            ok = np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
            assert ok, "T=%d E=%d Kr=%d K=%d N=%d w32=%s bits=(%d,%d) c=%d call %d plan %s" % (T, E, Kr, Kd, N, w32, bits_a, bits_w, c, rep, K.gemm_last_plan())


@pytest.mark.parametrize("w32", [False, True])
def test_moe_experts(K, oracle, w32):
    """routed experts end to end (dispatch, gather, grouped gate/up GEMMs, SiLU gate, grouped down GEMM, weighted
    combine) against the reference's loop over the experts restated on the oracle"""
    rng = np.random.default_rng(11 + w32)
    T, E, Kr, dim, inter = 40, 8, 3, 96, 160
    idx = _routing(rng, T, E, Kr)
    x = rand_i64(rng, (T, dim), 24)
    wts = rng.integers(1, 1 << 23, size=(T, Kr), dtype=np.int64)
    mk = (lambda shape: rand_i32(rng, shape, 27)) if w32 else (lambda shape: rand_i64(rng, shape, 27))
    w1, w3, w2 = [mk((inter, dim)) for _ in range(E)], [mk((inter, dim)) for _ in range(E)], [mk((dim, inter)) for _ in range(E)]
    d1, d3, d2 = [dev(w) for w in w1], [dev(w) for w in w3], [dev(w) for w in w2]
    y = K.moe_experts(dev(x), dev(wts), dev(idx), K.pointer_table(d1), K.pointer_table(d3), K.pointer_table(d2), w32, inter, 29, 27)
    ye = oracle.moe_experts(x, wts, idx, w1, w3, w2, 29, 27)
    assert np.array_equal(host(y), ye)


def test_witness_dump_writer(K, tmp_path):
    """saveTensor through the library's writer: same bytes as the reference's t.cpu().numpy().tobytes(), for device and
    host tensors, views, large tensors (several staging pieces) and many small files; a tensor overwritten right
    after the call still lands in the file with the contents it had at the call"""
    g = torch.Generator(device="cpu").manual_seed(9)
    cases = {
        "scores.bin": torch.randint(-(1 << 62), 1 << 62, (3, 5, 7, 11), generator=g).cuda(),
        "weights_u32.bin": torch.randint(-(1 << 31), 1 << 31, (129, 37), generator=g).to(torch.int32).cuda().view(torch.int32),
        "strided.bin": torch.randint(-9, 9, (64, 48), generator=g).cuda()[:, ::3],
        "host.bin": torch.randint(-9, 9, (1000,), generator=g),
        "big.bin": torch.randint(-(1 << 62), 1 << 62, ((13 << 20) + 5,), generator=g).cuda(),          # 104 MB: four pieces
    }
    want = {k: v.detach().cpu().contiguous().numpy().tobytes(order="C") for k, v in cases.items()}
    for name, t in cases.items():
        K.saveTensor(str(tmp_path / name), t)
    cases["big.bin"].zero_()                                   # queued behind the copy
    cases["scores.bin"].fill_(7)
    small = [torch.full((17,), i, dtype=torch.int64, device="cuda") for i in range(100)]
    for i, t in enumerate(small):
        K.saveTensor(str(tmp_path / ("small_%d.bin" % i)), t)
        t.add_(1000)
    K.dump_flush()
    for name, b in want.items():
        assert (tmp_path / name).read_bytes() == b, name
    for i in range(100):
        assert (tmp_path / ("small_%d.bin" % i)).read_bytes() == np.full(17, i, np.int64).tobytes()
    K.saveTensor(str(tmp_path / "missing_dir" / "x.bin"), small[0])
    with pytest.raises(RuntimeError):
        K.dump_flush()
    K.lib.zk_clear_error()


def test_converters(K, oracle):
    """the three float -> fixed converters the reference exports (inference/int64_gemm.cu:92-221)"""
    rng = np.random.default_rng(31)
    bits32 = rng.integers(0, 1 << 32, size=(37, 129), dtype=np.uint64).astype(np.uint32)
    bits16 = rng.integers(0, 1 << 16, size=(37, 129), dtype=np.uint64).astype(np.uint16)
    for rescale in (0, 12, 25, 40):
        o64 = torch.empty((37, 129), dtype=torch.int64, device="cuda")
        src = torch.from_numpy(bits32.view(np.int32)).cuda()
        K.lib.float32_to_int64_2d(src.data_ptr(), o64.data_ptr(), 37, 129, rescale)
        assert np.array_equal(host(o64), oracle.float32_to_int64_2d(bits32, rescale))
        o32 = torch.empty((37, 129), dtype=torch.int32, device="cuda")
        src16 = torch.from_numpy(bits16.view(np.int16)).cuda()
        K.lib.bf16_to_int32_2d(src16.data_ptr(), o32.data_ptr(), 37, 129, rescale)
        assert np.array_equal(host(o32), oracle.bf16_to_int32_2d(bits16, rescale))
    o32 = torch.empty((37, 129), dtype=torch.int32, device="cuda")
    K.lib.wkv_b_bf16_to_int32(src16.data_ptr(), o32.data_ptr(), 37, 129)
    assert np.array_equal(host(o32), oracle.wkv_b_bf16_to_int32(bits16))
    # pointers that are not 16-byte aligned take the scalar kernels; a length that is no multiple of the vector
    # width ends in a scalar tail
    big16 = torch.from_numpy(np.concatenate([bits16.ravel(), bits16.ravel()[:7]]).view(np.int16)).cuda()
    out = torch.empty((big16.numel(),), dtype=torch.int32, device="cuda")
    n = big16.numel() - 1
    K.lib.bf16_to_int32_2d(big16.data_ptr() + 2, out.data_ptr() + 4, 1, n, 12)
    want = oracle.bf16_to_int32_2d(big16.cpu().numpy().view(np.uint16)[1:].reshape(1, n), 12)
    assert np.array_equal(host(out)[1:], want.ravel())
    big32 = torch.from_numpy(np.concatenate([bits32.ravel(), bits32.ravel()[:3]]).view(np.int32)).cuda()
    out64 = torch.empty((big32.numel(),), dtype=torch.int64, device="cuda")
    n = big32.numel() - 1
    K.lib.float32_to_int64_2d(big32.data_ptr() + 4, out64.data_ptr() + 8, 1, n, 12)
    want = oracle.float32_to_int64_2d(big32.cpu().numpy().view(np.uint32)[1:].reshape(1, n), 12)
    assert np.array_equal(host(out64)[1:], want.ravel())
    K._check("converters")


@pytest.mark.parametrize("shape", [(256, 256), (300, 520), (1, 129), (129, 1), (7, 2048), (2048, 7168)])
def test_fp8_checkpoint_quantisation(K, oracle, shape):
    """block-scaled fp8 weights -> int32 fixed point in one pass (convert2.py:144-147): every fp8 code incl. NaN,
    scales from 2^-20 to 4, ragged block edges, values that saturate"""
    rows, cols = shape
    rng = np.random.default_rng(rows + cols)
    w = rng.integers(0, 256, (rows, cols), dtype=np.uint8)
    w[0, : min(cols, 256)] = np.arange(min(cols, 256), dtype=np.uint8)
    sc = np.exp2(rng.uniform(-20, 2, ((rows + 127) // 128, (cols + 127) // 128))).astype(np.float32)
    wd, sd = dev(w), dev(sc)
    for k in ((0, 21, 30) if rows * cols < (1 << 22) else (30,)):
        assert np.array_equal(host(K.quantize_fp8_weight(wd, sd, k)), oracle.fp8_block_scaled_to_int32(w, sc, k))
    assert np.array_equal(host(K.quantize_fp8_weight(wd.view(torch.float8_e4m3fn), sd, 25)), oracle.fp8_block_scaled_to_int32(w, sc, 25))


def test_bf16_checkpoint_quantisation(K, oracle):
    """(p.float() * 2^k).round() to int32 / int64 for every bfloat16 pattern (convert2.py:250-262, 290-295)"""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    pd = dev(bits.view(np.int16)).view(torch.bfloat16)
    for k in (0, 1, 15, 21, 31, 43, 127):
        assert np.array_equal(host(K.quantize_bf16(pd, k, torch.int32)), oracle.bf16_scaled_round(bits, k, np.int32))
        assert np.array_equal(host(K.quantize_bf16(pd, k, torch.int64)), oracle.bf16_scaled_round(bits, k, np.int64))
    out = torch.empty((4,), dtype=torch.int32, device="cuda")
    K.lib.bf16_scaled_round_to_int32(pd.data_ptr(), out.data_ptr(), 4, 128)
    assert K.lib.zk_last_error() == 1
    K.lib.zk_clear_error()


@pytest.mark.parametrize("seed", range(10 * SEEDS))
def test_rowwise_kernels_seeded_random_problems(K, oracle, seed):
    """softmax, activations and RMSNorm on random row lengths, row counts, magnitudes and weight types"""
    rng = np.random.default_rng(9800 + seed)
    for _ in range(4):
        T = int(rng.integers(1, 6000))
        rows = int(rng.integers(1, 40))
        fn, Q = [("softmax_q19", 19), ("softmax_q21", 21)][int(rng.integers(0, 2))]
        x = _scores(rng, (1, rows, 1, T), Q)
        if rng.integers(0, 2):
            x[0, :, 0, T // 2:] += -(64 << 36)                   # a masked tail
        R, C = dev(x), torch.empty((1, rows, 1, T), dtype=torch.int64, device="cuda")
        getattr(K, fn)(R, C)
        assert np.array_equal(host(C), getattr(oracle, fn)(x)[0]), "%s T=%d rows=%d" % (fn, T, rows)
        fn, Q = ACTS[int(rng.integers(0, 4))]
        shape = (1, int(rng.integers(1, 50)), int(rng.integers(1, 5000)))
        span = int(rng.choice([1, 8, 27, 70]))
        a = rng.integers(-(span << Q), span << Q, size=shape, dtype=np.int64)
        R, C = dev(a), torch.empty(shape, dtype=torch.int64, device="cuda")
        getattr(K, fn)(R, C)
        assert np.array_equal(host(C), getattr(oracle, fn)(a)), "%s shape=%s span=%d" % (fn, shape, span)
        N = int(rng.integers(1, 20001))
        M = int(rng.integers(1, 6))
        bits = int(rng.choice([8, 20, 31, 37, 50, 63]))
        A = rand_i64(rng, (M, N), bits)
        W = rng.integers(1, 1 << 20, size=(N,), dtype=np.int32) if rng.integers(0, 2) else rand_i64(rng, (N,), int(rng.choice([10, 40, 62])))
        Cn, rms = K.RMS_Norm_int64(dev(A), dev(W), 1, N)
        Ce, rmse = oracle.RMS_Norm_int64(A, W, 1, N)
        assert np.array_equal(rms[:M].numpy(), rmse) and np.array_equal(host(Cn), Ce), "rmsnorm M=%d N=%d bits=%d %s" % (M, N, bits, W.dtype)

