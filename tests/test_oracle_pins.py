"""Pins the CPU oracle BEFORE anything is compared against it.

The reference ships no tests or vectors for these kernels, so each oracle
function is held against (a) the tables/constants the reference's proving
circuits hold (tests/golden/zk_tables.json), (b) exact big-integer brute force
on tiny inputs, (c) library routines where the arithmetic coincides
(numpy int64 matmul, math.isqrt), and (d) closed forms / invariants that a
dropped term, wrong sign, wrong index or transposed operand would break.
"""
import math

import numpy as np
import pytest

from util import rand_i32, rand_i64, tdiv, wrap64, wrap128


# ----------------------------------------------------------------- tables ---
def test_lut_q19_q23_equal_reference_circuit_tables(oracle, zk_tables):
    assert oracle.softmax_init_q19().tolist() == zk_tables["q19Table"]
    assert oracle.silu_init_q23().tolist() == zk_tables["q23Table"]


@pytest.mark.parametrize("name,Q,sign", [("softmax_init_q19", 19, -1), ("softmax_init_q21", 21, -1),
                                         ("silu_init_q23", 23, 1), ("silu_init_q25", 25, 1)])
def test_lut_is_floor_of_exact_power(oracle, name, Q, sign):
    """LUT[i] = floor(2^Q * 2^(sign*i/256))  <=>  LUT^256 <= 2^(256Q + sign*i) < (LUT+1)^256, in exact integers."""
    lut = getattr(oracle, name)().tolist()
    for i, v in enumerate(lut):
        target = 1 << (256 * Q + sign * i)
        assert v ** 256 <= target < (v + 1) ** 256, (name, i, v)


def test_log2e_constants(zk_tables):
    for Q, c in ((19, zk_tables["LOG2E_Q19"]), (23, zk_tables["LOG2E_Q23"]), (21, 3025551), (25, 48408813)):
        assert c == round(math.log2(math.e) * 2 ** Q)


# ------------------------------------------------------------------- GEMM ---
def _gemm_bigint(A, W, a_rs, b_rs, c, init=0):
    Bd, M, K = A.shape
    N = W.shape[0]
    C = np.empty((Bd, M, N), np.int64)
    R = np.empty((Bd, M, N), np.int64)
    for b in range(Bd):
        for m in range(M):
            for n in range(N):
                s = init
                for k in range(K):
                    s += tdiv(int(A[b, m, k]), a_rs) * tdiv(int(W[n, k]), b_rs)
                s = wrap128(s)
                C[b, m, n] = wrap64(s >> c)
                R[b, m, n] = wrap64(s & ((1 << c) - 1))
    return C, R


@pytest.mark.parametrize("c", [0, 1, 29, 31, 33, 63])
@pytest.mark.parametrize("w32", [False, True])
def test_gemm_full_range_vs_bigint(oracle, c, w32):
    rng = np.random.default_rng(100 + c)
    A = rand_i64(rng, (2, 3, 37), 63)
    W = rand_i32(rng, (5, 37)) if w32 else rand_i64(rng, (5, 37), 63)
    A[0, 0, 0] = -(1 << 63)
    A[1, 2, 5] = (1 << 63) - 1
    C, R = oracle.int64_bmm_broadcast(A, W, 1, 1, c)
    Ce, Re = _gemm_bigint(A, W, 1, 1, c)
    assert np.array_equal(C, Ce) and np.array_equal(R, Re)


def test_gemm_rescale_truncates_toward_zero(oracle):
    rng = np.random.default_rng(7)
    A = rand_i64(rng, (1, 4, 19), 40)
    W = rand_i64(rng, (6, 19), 30)
    for a_rs, b_rs in ((1, 256), (3, 1), (-7, 5)):
        C, R = oracle.int64_bmm_broadcast(A, W, a_rs, b_rs, 11)
        Ce, Re = _gemm_bigint(A, W, a_rs, b_rs, 11)
        assert np.array_equal(C, Ce) and np.array_equal(R, Re)


def test_gemm_matches_numpy_when_nothing_overflows(oracle):
    """config-1 ranges: |sum| < 2^49, so int64 matmul followed by >> c is the same function."""
    rng = np.random.default_rng(1)
    A = rand_i64(rng, (1, 16, 512), 20)
    W = rand_i64(rng, (24, 512), 16)
    for c in (0, 29):
        C, R = oracle.int64_bmm_broadcast(A, W, 1, 1, c)
        full = A[0] @ W.T
        assert np.array_equal(C[0], full >> c)
        assert np.array_equal(C[0] * (1 << c) + R[0], full)       # X.W = C*2^c + R  (zk/src/index.ts:1948)
        assert (R >= 0).all() and (R < (1 << c) if c else R == 0).all()


def test_gemm_c0_full_range_is_wrapping_int64_matmul(oracle):
    rng = np.random.default_rng(2)
    A = rand_i64(rng, (1, 8, 64), 63)
    W = rand_i64(rng, (8, 64), 63)
    C, _ = oracle.int64_bmm_broadcast(A, W, 1, 1, 0)
    with np.errstate(over="ignore"):
        assert np.array_equal(C[0], A[0] @ W.T)


def test_gemm_operand_roles_not_transposed(oracle):
    A = np.zeros((1, 2, 3), np.int64)
    W = np.zeros((4, 3), np.int64)
    A[0, 1, 2] = 5
    W[3, 2] = 7
    C, _ = oracle.int64_bmm_broadcast(A, W, 1, 1, 0)
    exp = np.zeros((1, 2, 4), np.int64)
    exp[0, 1, 3] = 35
    assert np.array_equal(C, exp)


# ----------------------------------------------------------------- einsum ---
def _obj(x):
    return x.astype(object)


def _fin(s, rescale, init):
    f = np.vectorize(lambda v: wrap64(wrap128(int(v) + init) >> rescale), otypes=[np.int64])
    return f(s)


@pytest.mark.parametrize("bits,rescale", [(63, 23), (63, 0), (30, 21), (63, 37)])
def test_einsums_vs_object_einsum(oracle, bits, rescale):
    rng = np.random.default_rng(bits + rescale)
    B, S, H, D, Cc, T = 2, 3, 4, 5, 6, 7
    q = rand_i64(rng, (B, S, H, D), bits)
    w1 = rand_i32(rng, (H, D, Cc))
    assert np.array_equal(oracle.einsum_bshd_hdc_bshc(q, w1, rescale),
                          _fin(np.einsum("bshd,hdc->bshc", _obj(q), _obj(w1)), rescale, rescale // 2))
    a = rand_i64(rng, (B, S, H, Cc), bits)
    kv = rand_i64(rng, (B, T, Cc), bits)
    assert np.array_equal(oracle.einsum_bshc_btc_bsht(a, kv, rescale),
                          _fin(np.einsum("bshc,btc->bsht", _obj(a), _obj(kv)), rescale, rescale // 2))
    p = rand_i64(rng, (B, S, H, T), bits)
    assert np.array_equal(oracle.einsum_bsht_btc_bshc(p, kv, rescale),
                          _fin(np.einsum("bsht,btc->bshc", _obj(p), _obj(kv)), rescale, rescale // 2))
    w2 = rand_i32(rng, (H, D, Cc))
    assert np.array_equal(oracle.einsum_bshc_hdc_bshd(a, w2, rescale),
                          _fin(np.einsum("bshc,hdc->bshd", _obj(a), _obj(w2)), rescale, 0))     # no rounding term


def test_einsum_rounding_term_is_half_the_shift_count(oracle):
    """inference/int64_gemm.cu:442: init = rescale/2 (e.g. 11 for 23), not 2^(rescale-1)."""
    a = np.zeros((1, 1, 1, 2), np.int64)
    b = np.zeros((1, 1, 2), np.int64)
    a[0, 0, 0, 0] = (1 << 23) - 11
    b[0, 0, 0] = 1
    assert oracle.einsum_bshc_btc_bsht(a, b, 23)[0, 0, 0, 0] == 1      # (2^23 - 11 + 11) >> 23
    a[0, 0, 0, 0] -= 1
    assert oracle.einsum_bshc_btc_bsht(a, b, 23)[0, 0, 0, 0] == 0


def test_each_einsum_has_its_own_rounding_term(oracle):
    """one product of 1 * v per output, so the sum is v: the first three einsums add rescale/2 = 11 before >> 23
    (inference/int64_gemm.cu:401, :442, :483), the fourth adds nothing (:525)"""
    v = (1 << 23) - 11
    for below in (0, 1):
        a = np.full((1, 1, 1, 1), v - below, np.int64)
        assert oracle.einsum_bshd_hdc_bshc(a, np.ones((1, 1, 1), np.int32), 23)[0, 0, 0, 0] == 1 - below
        assert oracle.einsum_bshc_btc_bsht(a, np.ones((1, 1, 1), np.int64), 23)[0, 0, 0, 0] == 1 - below
        assert oracle.einsum_bsht_btc_bshc(a, np.ones((1, 1, 1), np.int64), 23)[0, 0, 0, 0] == 1 - below
        assert oracle.einsum_bshc_hdc_bshd(a, np.ones((1, 1, 1), np.int32), 23)[0, 0, 0, 0] == 0
    a = np.full((1, 1, 1, 1), 1 << 23, np.int64)
    assert oracle.einsum_bshc_hdc_bshd(a, np.ones((1, 1, 1), np.int32), 23)[0, 0, 0, 0] == 1
    assert oracle.einsum_bshc_hdc_bshd(a - 1, np.ones((1, 1, 1), np.int32), 23)[0, 0, 0, 0] == 0


# ------------------------------------------------------------------- RoPE ---
def test_rope_identity_and_bigint(oracle):
    rng = np.random.default_rng(5)
    A = rand_i64(rng, (2, 3, 4, 8, 2), 63)
    ident = np.zeros((1, 3, 1, 8, 2), np.int64)
    ident[..., 0] = 1 << 42
    assert np.array_equal(oracle.complex_int64_mul_broadcast(A, ident), A)      # times (1 + 0i)
    Bt = rand_i64(rng, (1, 3, 1, 8, 2), 43)
    out = oracle.complex_int64_mul_broadcast(A, Bt)
    for idx in np.ndindex(2, 3, 4, 8):
        b, s, h, d = idx
        a0, a1 = int(A[b, s, h, d, 0]), int(A[b, s, h, d, 1])
        b0, b1 = int(Bt[0, s, 0, d, 0]), int(Bt[0, s, 0, d, 1])
        p = lambda x, y: wrap64((x * y) >> 42)          # floor division by 2^42 (zk/src/index.ts:2212-2256)
        assert out[b, s, h, d, 0] == wrap64(p(a0, b0) - p(a1, b1))
        assert out[b, s, h, d, 1] == wrap64(p(a0, b1) + p(a1, b0))


def test_rope_close_to_float_rotation(oracle):
    rng = np.random.default_rng(6)
    A = rand_i64(rng, (1, 5, 2, 4, 2), 31)
    ang = rng.uniform(0, 2 * math.pi, size=(1, 5, 1, 4))
    Bt = np.stack([np.round(np.cos(ang) * 2 ** 42), np.round(np.sin(ang) * 2 ** 42)], -1).astype(np.int64)
    out = oracle.complex_int64_mul_broadcast(A, Bt)
    z = (A[..., 0] + 1j * A[..., 1]) * np.exp(1j * ang)
    assert np.abs(out[..., 0] - z.real).max() < 4 and np.abs(out[..., 1] - z.imag).max() < 4


# ---------------------------------------------------------------- RMSNorm ---
@pytest.mark.parametrize("bits", [20, 37, 63])
def test_rms_stat_is_isqrt(oracle, bits):
    rng = np.random.default_rng(bits)
    A = rand_i64(rng, (5, 7168), bits)
    if bits == 63:
        A[0, :] = (1 << 63) - 1        # sum ~ 7168 * 2^126 ~ 2^138.8: needs the 192-bit accumulator
    rms = oracle.rms_stat(A, 1, 7168)
    for m in range(5):
        acc = 1 + sum(int(v) * int(v) for v in A[m])
        q = acc // 7168
        assert rms[m] == math.isqrt(q)
        assert int(rms[m]) ** 2 <= q < (int(rms[m]) + 1) ** 2        # zk/src/index.ts:989-996


def test_rms_stat_adds_eps_before_dividing(oracle):
    """inference/kernel.py:477-494: (eps + sum a^2) // dim.  Row [1,1,1,0] with dim 4: (1 + 3) // 4 = 1 -> rms 1; a
    statistic that drops eps gets 3 // 4 = 0.  Row of four 3s with dim 4: (1 + 36) // 4 = 9 -> 3; dividing by dim - 1 or
    rounding up would not."""
    A = np.array([[1, 1, 1, 0], [3, 3, 3, 3], [2, 2, 2, 1]], np.int64)
    assert oracle.rms_stat(A, 1, 4).tolist() == [1, 3, 1]            # (1 + 13) // 4 = 3 -> isqrt 1
    assert oracle.rms_stat(A, 3, 4).tolist() == [1, 3, 2]            # (3 + 13) // 4 = 4 -> 2


@pytest.mark.parametrize("w32", [True, False])
def test_rms_apply_is_floor_division(oracle, w32):
    rng = np.random.default_rng(11)
    A = rand_i64(rng, (3, 64), 63)
    W = rand_i32(rng, (64,)) if w32 else rand_i64(rng, (64,), 63)
    rms = np.array([1, 12345678901, (1 << 62) + 12345], np.int64)
    C = oracle.rms_norm_apply(A, W, rms)
    for m in range(3):
        for n in range(64):
            assert C[m, n] == wrap64((int(A[m, n]) * int(W[n])) // int(rms[m]))      # Python // is floor


# ---------------------------------------------------------------- softmax ---
def _ref_float_softmax(x, Q):
    xf = x.astype(np.float64) / 2 ** Q
    e = np.exp(xf - xf.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


@pytest.mark.parametrize("fn,Q", [("softmax_q19", 19), ("softmax_q21", 21)])
def test_softmax_invariants_and_float(oracle, fn, Q):
    rng = np.random.default_rng(Q)
    x = rng.integers(-(8 << Q), 8 << Q, size=(2, 3, 4, 257), dtype=np.int64)
    C, w = getattr(oracle, fn)(x)
    assert (C >= 0).all() and (C <= (1 << Q)).all()
    assert (C.sum(-1) <= (1 << Q) + (128 if Q == 21 else 0)).all()          # q21 rounds, q19 truncates
    assert np.abs(C / 2 ** Q - _ref_float_softmax(x, Q)).max() < 4e-3       # LUT has 8 fractional bits
    am = x.argmax(-1)
    sw = w.sum(-1)
    top = np.take_along_axis(C, am[..., None], -1)[..., 0]
    if Q == 19:
        assert np.array_equal(top, (1 << 38) // sw)                          # max element has w = LUT[0] = 2^19
    else:
        assert np.array_equal(top, ((1 << 42) + sw // 2) // sw)


def test_softmax_q19_uniform_row_and_mask(oracle):
    for n in (1, 3, 7, 1024):
        x = np.full((1, 1, 1, n), 12345, np.int64)
        C, w = oracle.softmax_q19(x)
        assert (w == 1 << 19).all() and (C == (1 << 19) // n).all()
    x = np.zeros((1, 1, 1, 8), np.int64)
    x[..., 4:] = -(1 << 42)                       # the causal mask value (inference/model.py:1555)
    C, w = oracle.softmax_q19(x)
    assert C[0, 0, 0].tolist() == [1 << 17] * 4 + [0] * 4
    x = np.array([0, -(1 << 25), -(1 << 25) - 1], np.int64).reshape(1, 1, 1, 3)      # clip is d > 2^25, exclusive
    _, w = oracle.softmax_q19(x)
    assert w[0, 0, 0].tolist() == [1 << 19, 0, 0]          # d = 2^25 passes the clip but k = 92 >= 64


def test_softmax_q19_single_element_steps(oracle):
    """hand-computed from the definition: d=2^19 (x = max - 1.0): y = 756388, k = 1, f = 232100, LUT[113] >> 1."""
    x = np.array([0, -(1 << 19)], np.int64).reshape(1, 1, 1, 2)
    C, w = oracle.softmax_q19(x)
    # worked by hand from inference/int64_gemm.cu:700-708 and the table the circuits hold (zk/src/index.ts:2645-2681):
    # y = (2^19 * 756388) >> 19 = 756388, k = 1, f = 232100, index 113, entry 386095, w = 386095 >> 1
    assert w[0, 0, 0].tolist() == [524288, 193047]
    assert C[0, 0, 0].tolist() == [383193, 141094]          # floor(w * 2^19 / (524288 + 193047))
    assert abs(w[0, 0, 0, 1] / 2 ** 19 - math.exp(-1)) < 2e-3


def test_softmax_q21_hand_steps_rounded_exponent_and_rounded_quotient(oracle):
    """Worked by hand from inference/int64_gemm.cu:624-657 at inputs where each rounding decides the result.

    Row [0, -11356, -2924304] (max 0, so d = x).  LOG2E_Q21 = 3025551, 2^21 = 2097152, 2^20 = 1048576.
    d = -11356:   d*L = -34358157156.  -16384*2^21 = -34359738368 < d*L < -16383*2^21 = -34357641216, and
                  d*L + 2^20 = -34357108580 > -16383*2^21, so y = -16383 (:634; WITHOUT the + 2^20 it is -16384).
                  -y = 16383: k = 0, f = 16383, f >> 13 = 1 (:636-641; 16384 >> 13 would be 2), w = LUT[1].
    d = -2924304: d*L = -8847630891504 = -4218879.2.. * 2^21, + 2^20 -> y = -4218879 (floor alone: -4218880).
                  -y = 4218879 = 2*2^21 + 24575: k = 2, f = 24575, f >> 13 = 2 (24576 >> 13 would be 3), w = LUT[2] >> 2.
    LUT[i] = floor(2^21 * 2^(-i/256)) (:672-680): LUT[1] = 2091481, LUT[2] = 2085826 -- the reference holds no copy of
    this table, so the two literals are checked below by the exact inequality v^256 <= 2^(256*21 - i) < (v+1)^256.
    w = [2097152, 2091481, 521456], sumW = 4710089, sumW/2 = 2355044 (:656-657):
      (2097152*2^21 + 2355044) / 4710089 = 933750      (without the + sumW/2: 933750)
      (2091481*2^21 + 2355044) / 4710089 = 931225      (931225)
      ( 521456*2^21 + 2355044) / 4710089 = 232177      (232176: the rounding of the quotient decides)"""
    for i, v in ((1, 2091481), (2, 2085826)):
        assert v ** 256 <= 1 << (256 * 21 - i) < (v + 1) ** 256
    assert oracle.softmax_init_q21()[:3].tolist() == [2097152, 2091481, 2085826]
    x = np.array([0, -11356, -2924304], np.int64).reshape(1, 1, 1, 3)
    C, w = oracle.softmax_q21(x)
    assert w[0, 0, 0].tolist() == [2097152, 2091481, 521456]
    assert C[0, 0, 0].tolist() == [933750, 931225, 232177]
    # the same arithmetic in exact integers, so that the literals above are not only the oracle's word
    assert -16384 * 2097152 < -11356 * 3025551 < -16383 * 2097152 < -11356 * 3025551 + 1048576
    assert -4218880 * 2097152 < -2924304 * 3025551 < -4218879 * 2097152 < -2924304 * 3025551 + 1048576
    assert 4218879 == 2 * 2097152 + 24575 and 2 * 8192 <= 24575 < 3 * 8192 and 2085826 // 4 == 521456
    s = 2097152 + 2091481 + 521456
    assert 232177 * s <= 521456 * 2097152 + s // 2 < 232178 * s and 521456 * 2097152 < 232177 * s


def test_softmax_clips_decide_for_distances_beyond_the_products_width(oracle):
    """The clips (inference/int64_gemm.cu:706 `d > 64<<19`, :627 `d < -(64<<21)`) change nothing for moderate distances
    (there k >= 64 or the table entry shifted by k >= 22 is 0 anyway: at d = 2^25 resp. -2^27 exactly both branches give
    0, so `>` against `>=` cannot be told apart by any input), but they are what keeps a masked element at 0 once the
    product leaves its width: q21 multiplies in 64 bits (:634), and -2^42 * 3025551 = -1.33e19 wraps to a positive y,
    which without the clip indexes the table with a negative k; q19's y is the low 64 bits of a 128-bit product (:713),
    negative for d = 2^63."""
    x = np.array([0, -(1 << 42)], np.int64).reshape(1, 1, 1, 2)           # the causal mask value, inference/model.py:1555
    C, w = oracle.softmax_q21(x)
    assert w[0, 0, 0].tolist() == [1 << 21, 0] and C[0, 0, 0].tolist() == [1 << 21, 0]
    for lo in (-(1 << 62), -(1 << 62) - 12345, -(1 << 63) + (1 << 62) - 99):
        x = np.array([1 << 62, lo, (1 << 62) - 1], np.int64).reshape(1, 1, 1, 3)
        C, w = oracle.softmax_q19(x)
        assert w[0, 0, 0, :2].tolist() == [1 << 19, 0] and C[0, 0, 0, 1] == 0
    x = np.array([(1 << 62), -(1 << 62), -(1 << 61)], np.int64).reshape(1, 1, 1, 3)
    C, w = oracle.softmax_q21(x)
    assert w[0, 0, 0].tolist() == [1 << 21, 0, 0]
    # d = -ceil(2^64 / 3025551) = -6096986655889 (about 1.4 times the mask value): d * L = -(2^64 + 2068223) wraps to
    # -2068223, whose y = -1 would index the table at k = 0 and give w = 2^21, as much as the maximum itself
    assert 6096986655889 * 3025551 == (1 << 64) + 2068223
    x = np.array([0, -6096986655889], np.int64).reshape(1, 1, 1, 2)
    C, w = oracle.softmax_q21(x)
    assert w[0, 0, 0].tolist() == [1 << 21, 0] and C[0, 0, 0].tolist() == [1 << 21, 0]


# ------------------------------------------------------------- activations ---
@pytest.mark.parametrize("Q", [23, 25])
def test_sigmoid_silu_special_values_and_float(oracle, Q):
    sig = getattr(oracle, "sigmoid_q%d" % Q)
    silu = getattr(oracle, "silu_q%d" % Q)
    one = 1 << Q
    x = np.array([0, 64 * one, -64 * one, 64 * one - 1, -64 * one + 1, 100 * one], np.int64)
    s = sig(x)
    assert s[0] == one // 2 and s[1] == 64 * one and s[2] == 0 and s[5] == 100 * one      # returns x above the limit
    assert s[3] == one
    # x just above -64: k = 92 >= 64, the clamped shift makes u = 0 and sigma = 1.0 (hardware-defined corner of
    # inference/int64_gemm.cu:1008, fixed here as NVIDIA's clamped shift; parity unpinned)
    assert s[4] == one
    assert silu(x)[0] == 0 and silu(x)[1] == 64 * one and silu(x)[2] == 0
    rng = np.random.default_rng(Q)
    x = rng.integers(-20 * one, 20 * one, size=(4096,), dtype=np.int64)
    xf = x / one
    sf = 1 / (1 + np.exp(-xf))
    assert np.abs(sig(x) / one - sf).max() < 2e-3
    assert np.abs(silu(x) / one - xf * sf).max() < 2e-2
    assert np.abs((sig(x) + sig(-x)) / one - 1).max() < 4e-3                               # sigma(x)+sigma(-x) = 1
    assert (np.diff(sig(np.sort(x))) >= -(one >> 8)).all()                                 # monotone up to LUT steps


def test_sigmoid_q23_hand_steps(oracle):
    """x = -1.0: y = (2^23 * 12102203) >> 23 = 12102203; k = 1, f = 3713595, t = LUT[113]; u = t << 1."""
    # literals worked by hand from inference/int64_gemm.cu:932-945 with the table the circuits hold
    # (zk/src/index.ts:3382-3418): index 113, entry 11391119, u = 22782238, 2^46 // (2^23 + u)
    x = np.array([-(1 << 23)], np.int64)
    assert oracle.sigmoid_q23(x)[0] == 2257517
    assert oracle.silu_q23(x)[0] == (-(1 << 23) * 2257517) >> 23 == -2257517
    # x = -22713: (-x) * L = 274877336739 < 2^38 = 274877906944, so y = 32767, table cell 0, u = 2^23, q = 2^46 / 2^24.
    # Negating AFTER the shift (as q25 does, :804) gives -floor(-32767.9..) = 32768: cell 1, q = 4188625.
    assert 22713 * 12102203 == 274877336739 < 1 << 38
    x = np.array([-22713], np.int64)
    assert oracle.sigmoid_q23(x)[0] == 1 << 22
    assert oracle.silu_q23(x)[0] == -11357                  # floor(-22713 * 2^22 / 2^23) = floor(-11356.5)
    # q23 negates before the shift, q25 after: they differ in rounding for positive inputs
    # x = 3, q23: y = (-3 * 12102203) >> 23 = -5, k = -1, f = 2^23 - 5, index 255; q25: y = -((3 * 48408813) >> 25) = -4
    x = np.array([3], np.int64)
    assert oracle.sigmoid_q23(x)[0] == 4199982
    assert oracle.sigmoid_q25(x)[0] == 16799929


def test_sigmoid_silu_q25_hand_steps_negation_after_the_shift(oracle):
    """Worked by hand from inference/int64_gemm.cu:804-818: y = -int64((r * 48408813) >> 25) floors BEFORE negating
    (q23 negates first, :932), which moves y by one whenever the product is not a multiple of 2^25.

    r = -90852: r*L = -4398037478676, and -2^42 = -4398046511104 < r*L < -131071 * 2^25 = -4398012956672, so the
    arithmetic shift gives -131072 and y = 131072 = 2^17: k = 0, f = 2^17, f >> 17 = 1, u = t = LUT25[1] = 33645407.
    (Negating first: (90852*L) >> 25 = 131071, f >> 17 = 0, t = 2^25, q = 2^50 / 2^26 = 16777216.)
    q = 2^50 / (2^25 + 33645407) = 1125899906842624 / 67199839 = 16754503;  SiLU = (r*q) >> 25 = floor(-45364.2) = -45365.
    r = 181705: r*L = 8796123366165 = 262144.9.. * 2^25, so y = -262144 (negating first: -262145): k = -1,
    f = 2^25 - 262144 = 33292288, f >> 17 = 254 (33292287 >> 17 = 253), u = LUT25[254] >> 1 = 66746437 >> 1 = 33373218,
    q = 2^50 / (2^25 + 33373218) = 16822642; SiLU = (181705 * 16822642) >> 25 = 91098.
    LUT25[i] = floor(2^25 * 2^(i/256)) (:832-839); the reference holds no copy, so the literals are checked exactly."""
    for i, v in ((1, 33645407), (254, 66746437)):
        assert v ** 256 <= 1 << (256 * 25 + i) < (v + 1) ** 256
    lut = oracle.silu_init_q25().tolist()
    assert lut[0] == 1 << 25 and lut[1] == 33645407 and lut[254] == 66746437
    assert -(1 << 42) < -90852 * 48408813 < -131071 * (1 << 25)
    assert 16754503 * 67199839 <= 1 << 50 < 16754504 * 67199839
    assert 262144 * (1 << 25) < 181705 * 48408813 < 262145 * (1 << 25)
    assert 16822642 * ((1 << 25) + 33373218) <= 1 << 50 < 16822643 * ((1 << 25) + 33373218)
    x = np.array([-90852, 181705], np.int64)
    assert oracle.sigmoid_q25(x).tolist() == [16754503, 16822642]
    assert oracle.silu_q25(x).tolist() == [-45365, 91098]
    assert -45365 * (1 << 25) <= -90852 * 16754503 < -45364 * (1 << 25)
    assert 91098 * (1 << 25) <= 181705 * 16822642 < 91099 * (1 << 25)
    # the same two inputs through q23's order of operations land one table cell away (what :932 against :804 means)
    assert oracle.sigmoid_q25(np.array([-407108648], np.int64))[0] == 180          # (r*L) >> 25 = -587333632, k = 17, cell 129


# -------------------------------------------------------------------- float -> fixed converters ---
def test_converters_truncate_the_scaled_float(oracle):
    """the converters scale the INTEGER mantissa (1.m * 2^23 for fp32, 1.m * 2^7 for bf16) by 2^(exp + rescale), so
    the value is trunc(|x| * 2^(rescale + 23)) resp. trunc(|x| * 2^(rescale + 7)) with the sign applied afterwards:
    checked against exact rational arithmetic wherever the 32-bit shift of the reference is defined"""
    from fractions import Fraction
    rng = np.random.default_rng(77)
    f = (rng.standard_normal(4000) * np.exp(rng.uniform(-12, 6, 4000))).astype(np.float32)
    f[:6] = [0.0, -0.0, 1.0, -1.0, 0.5, -0.4999]
    bits32 = f.view(np.uint32)
    checked = 0
    for rescale in (-20, -3, 0, 8):
        out = oracle.float32_to_int64_2d(bits32.reshape(40, 100), rescale).ravel()
        for x, o in zip(f.tolist(), out.tolist()):
            if x == 0:
                assert o == 0
                continue
            ex2 = int(np.frexp(np.float32(x))[1]) - 1 + rescale
            if -31 < ex2 < 31 and abs(x) >= 2.0 ** -126:
                want = int(abs(Fraction(x)) * Fraction(2) ** (rescale + 23))
                assert o == (want if x > 0 else -want), (x, rescale)
                checked += 1
    assert checked > 8000
    bf = (bits32 >> 16).astype(np.uint16)                          # truncating fp32 -> bf16 gives valid bf16 patterns
    fb = (bf.astype(np.uint32) << 16).view(np.float32)
    out = oracle.bf16_to_int32_2d(bf.reshape(40, 100), 12).ravel()
    for x, o in zip(fb.tolist(), out.tolist()):
        if x == 0:
            assert o == 0
            continue
        ex2 = int(np.frexp(np.float32(x))[1]) - 1 + 12
        if -31 < ex2 < 24 and abs(x) >= 2.0 ** -126:
            want = int(abs(Fraction(x)) * Fraction(2) ** (12 + 7))
            assert o == (want if x > 0 else -want), x
    sat = oracle.wkv_b_bf16_to_int32(bf.reshape(40, 100)).ravel()
    plain = oracle.bf16_to_int32_2d(bf.reshape(40, 100), 25).ravel()
    for x, o, pl in zip(fb.tolist(), sat.tolist(), plain.tolist()):
        if abs(x) >= 0.5:
            assert o == 0x7FFFFFFF                                 # saturates regardless of sign (:151-154)
        else:
            assert o == pl                                         # otherwise the rescale-25 conversion


# ------------------------------------------------------------------------------ gate routing ---
def _route_numpy(scores, bias, n_groups, topk_groups, topk):
    """independent restatement with numpy's sorts (stable, so ties go to the lower index)"""
    T, E = scores.shape
    sc = scores + (0 if bias is None else bias.astype(np.int64)[None, :])
    if n_groups > 1:
        grp = sc.reshape(T, n_groups, E // n_groups)
        srt = -np.sort(-grp, axis=-1)
        gscore = srt[..., :2].sum(-1) if bias is not None else srt[..., 0]
        gsel = np.argsort(-gscore, axis=-1, kind="stable")[:, :topk_groups]
        keep = np.zeros((T, n_groups), bool)
        np.put_along_axis(keep, gsel, True, axis=1)
        sc = np.where(np.repeat(keep, E // n_groups, axis=1), sc, -(1 << 42))
    idx = np.argsort(-sc, axis=-1, kind="stable")[:, :topk]
    raw = np.take_along_axis(scores, idx, axis=1)
    w = (raw * (1 << 23)) // raw.sum(-1, keepdims=True)
    return w * 5 // 2, idx, raw


def test_checkpoint_quantisation_equals_the_tensor_ops_it_restates(oracle):
    """fp8_block_scaled_to_int32 / bf16_scaled_round against torch's own CPU tensor ops, written as convert2.py writes
    them (inference/convert2.py:144-147, 250-262) with the Triton kernel's three operations (kernel.py:90-93: load
    as float32, multiply by the block scale, store as bfloat16) as tensor ops: every fp8 code, scales from tiny to
    large, ragged block edges, ties of both roundings."""
    import torch
    rng = np.random.default_rng(8)
    tab = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    mine = oracle._e4m3fn_table()
    assert np.array_equal(np.isnan(tab), np.isnan(mine)) and np.array_equal(tab[~np.isnan(tab)], mine[~np.isnan(mine)])
    for rows, cols in ((256, 256), (300, 520), (1, 129), (129, 1)):
        w = rng.integers(0, 256, (rows, cols), dtype=np.uint8)
        w[0, : min(cols, 256)] = np.arange(min(cols, 256), dtype=np.uint8)
        sc = np.exp2(rng.uniform(-20, 2, ((rows + 127) // 128, (cols + 127) // 128))).astype(np.float32)
        for k in (0, 7, 21, 30):
            x = torch.from_numpy(w).view(torch.float8_e4m3fn).to(torch.float32)
            s = torch.from_numpy(sc).repeat_interleave(128, 0).repeat_interleave(128, 1)[:rows, :cols]
            z = ((x * s).to(torch.bfloat16).to(torch.float32) * (2 ** k)).round()
            inside = (~torch.isnan(z)) & (z.abs() < 2.0 ** 31)
            want = z[inside].to(torch.int32).numpy()
            got = oracle.fp8_block_scaled_to_int32(w, sc, k)
            assert np.array_equal(got[inside.numpy()], want)
            assert np.all(got[torch.isnan(z).numpy()] == 0)
            assert np.all(got[(z >= 2.0 ** 31).numpy()] == 2 ** 31 - 1) and np.all(got[(z <= -(2.0 ** 31)).numpy()] == -(2 ** 31))
    # every bfloat16 pattern, both widths; k = 0 and 1 put values exactly on .5 (round half to even)
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    pt = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)
    for k in (0, 1, 15, 31, 43):
        z = (pt.to(torch.float32) * (2 ** k)).round()
        for dt, tdt, lim in ((np.int32, torch.int32, 2.0 ** 31), (np.int64, torch.int64, 2.0 ** 63)):
            inside = (~torch.isnan(z)) & (z.abs() < lim)
            got = oracle.bf16_scaled_round(bits, k, dt)
            assert np.array_equal(got[inside.numpy()], z[inside].to(tdt).numpy())
            assert np.all(got[torch.isnan(z).numpy()] == 0)
    assert oracle.bf16_scaled_round(np.array([0x3F00, 0x3FC0, 0x4020, 0xBF00, 0xBFC0], np.uint16), 0, np.int32).tolist() == [0, 2, 2, 0, -2]
    # ties of the bfloat16 store: 1 + 2^-8 is halfway between 1 and 1 + 2^-7 -> even (1); 1 + 3*2^-8 -> 1 + 2^-6
    y = oracle._round_to_bf16(np.array([1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8, -(1 + 2.0 ** -8)], np.float32))
    assert y.tolist() == [1.0, 1 + 2.0 ** -6, -1.0]


@pytest.mark.parametrize("E,G,KG,K", [(256, 8, 4, 8), (16, 4, 2, 4), (64, 1, 1, 6), (96, 3, 3, 5), (512, 8, 3, 8)])
@pytest.mark.parametrize("with_bias", [True, False])
def test_gate_route_matches_the_tensor_op_restatement(oracle, E, G, KG, K, with_bias):
    rng = np.random.default_rng(E + G + with_bias)
    scores = rng.integers(1, 1 << 23, size=(50, E), dtype=np.int64)            # sigmoid_q23 outputs
    bias = rng.integers(-(1 << 20), 1 << 20, size=E, dtype=np.int64).astype(np.int32) if with_bias else None
    w, idx, raw = oracle.gate_route(scores, bias, G, KG, K)
    we, ie, re_ = _route_numpy(scores, bias, G, KG, K)
    assert np.array_equal(idx, ie) and np.array_equal(raw, re_) and np.array_equal(w, we)
    # what the arithmetic fixes: winners are distinct, sorted by biased score, and the weights are Q23 shares * 2.5
    assert all(len(set(r)) == K for r in idx.tolist())
    assert np.all(w >= 0) and np.all(w.sum(-1) <= (5 << 23) // 2) and np.all(w.sum(-1) > ((5 << 23) // 2) - 3 * K)


def test_gate_route_hand_case_and_ties(oracle):
    """8 experts in 4 groups of 2, keep 2 groups, pick 3.  Biased scores by group: (10,1) (7,7) (9,3) (7,7): group
    scores 11, 14, 12, 14 -> groups 1 and 3 win (the tie between them does not matter), group 2 beats group 0 for
    nothing.  Among experts 2,3,6,7 all biased scores are 7: the lower indices win."""
    scores = np.array([[10, 1, 7, 7, 9, 3, 7, 7]], np.int64)
    w, idx, raw = oracle.gate_route(scores, np.zeros(8, np.int32), 4, 2, 3)
    assert idx.tolist() == [[2, 3, 6]] and raw.tolist() == [[7, 7, 7]]
    assert w.tolist() == [[((7 << 23) // 21) * 5 // 2] * 3]
    # the bias decides the routing but the weights come from the unbiased scores
    bias = np.array([0, 0, 0, 0, 100, 100, 0, 0], np.int32)
    w, idx, raw = oracle.gate_route(scores, bias, 4, 2, 3)
    assert idx.tolist() == [[4, 5, 2]] and raw.tolist() == [[9, 3, 7]]
    assert w.tolist() == [[((9 << 23) // 19) * 5 // 2, ((3 << 23) // 19) * 5 // 2, ((7 << 23) // 19) * 5 // 2]]
    # without a bias a group is scored by its maximum: 10, 7, 9, 7 -> groups 0 and 2
    w, idx, raw = oracle.gate_route(scores, None, 4, 2, 3)
    assert idx.tolist() == [[0, 4, 5]]


# ------------------------------------------------ the proving circuits' own restatement of the kernels ---
# zk/src/index.ts re-derives every kernel result inside the circuits: a proof only verifies if the witness the kernels
# wrote satisfies THESE formulas.  They are restated below in Python big integers, following the TypeScript (not the
# CUDA source the oracle follows), with the tables the circuits hold, and compared with the oracle on random inputs in
# the model's domain.
def ts_shr_var(x, k):
    """shrVar, zk/src/index.ts:2690-2706 / 3425-3440: a shift by the low six bits of k"""
    return x >> (k & 63)


def ts_softmax_row_q19(xs, table, log2e):
    """calcSumW (zk/src/index.ts:3058-3093) for the sum, the section circuit (:2721-2757) for the quotients"""
    xmax = max(xs)
    ws = []
    for x in xs:
        d = xmax - x
        if d > (64 << 19):                      # :3071 (the circuit has no such test: k >= 64 zeroes the same elements)
            ws.append(0)
            continue
        y = (d * log2e) >> 19                   # :3075, :2733
        k = y >> 19
        if k >= 64:                             # :3078, :2740
            ws.append(0)
            continue
        f = (y - k * (1 << 19)) >> (19 - 8)     # :3082, :2735
        ws.append(ts_shr_var(table[f], k))
    total = sum(ws)
    return ws, [0 if total == 0 else (w << 19) // total for w in ws]        # :2752-2753


def ts_sigmoid_q23(x, table, log2e):
    """the witness and the constraints of the sigmoid circuit, zk/src/index.ts:3511-3557"""
    pdt = -x * log2e                            # :3511
    q = pdt >> 23                               # :3519
    k = q >> 23                                 # :3521
    f = q & ((1 << 23) - 1)
    t = table[f >> (23 - 8)]                    # :3523-3525
    u = t >> (-k & 63) if k < 0 else (t << (k & 63)) & ((1 << 64) - 1)      # :3551 with shrVar / shlVar on UInt64
    if abs(k) >= 63:                            # :3553 (`Bool && Bool` in JavaScript yields its second operand)
        u = 0
    return (1 << 46) // ((1 << 23) + u)         # :3555


def test_softmax_q19_equals_the_circuits_restatement(oracle, zk_tables):
    table, log2e = zk_tables["q19Table"], zk_tables["LOG2E_Q19"]
    rng = np.random.default_rng(2721)
    rows = 0
    for T, n in ((1, 3000), (2, 2500), (3, 2000), (7, 1500), (31, 800), (64, 500), (128, 300), (200, 200)):
        x = rng.integers(-(12 << 19), 12 << 19, size=(1, 1, n, T), dtype=np.int64)
        if T > 1:
            # causal rows: a masked tail at -2^42 (inference/model.py:1555), and distances right at the clip
            for r in range(0, n, 3):
                x[0, 0, r, rng.integers(1, T):] = -(1 << 42)
            edge = rng.integers(0, n, size=n // 4)
            x[0, 0, edge, 0] = x[0, 0, edge].max(axis=1) - (1 << 25) - rng.integers(-2, 3, size=edge.size)
            x[0, 0, edge[::2], T - 1] = x[0, 0, edge[::2]].max(axis=1) - rng.integers(0, 1 << 25, size=edge[::2].size)
        C, W = oracle.softmax_q19(x)
        for r in range(n):
            ws, cs = ts_softmax_row_q19([int(v) for v in x[0, 0, r]], table, log2e)
            assert W[0, 0, r].tolist() == ws and C[0, 0, r].tolist() == cs, (T, r)
        rows += n
    assert rows >= 10000


def test_sigmoid_silu_q23_equal_the_circuits_restatement(oracle, zk_tables):
    """the quotient q = 2^46 // (2^23 + u) as the circuits constrain it, for k on both sides of 0, |x| up to the kernel's
    saturation limit on the positive side and down to -27.7 (beyond it `t << k` leaves 64 bits: hardware-defined in the
    CUDA build, parity unpinned).  SiLU is (x * q) >> 23 with that q (inference/int64_gemm.cu:945); the circuits write
    x.mul(q).div(2^23) (:3651), whose rounding for negative x is o1js's and is not pinned here."""
    table, log2e = zk_tables["q23Table"], zk_tables["LOG2E_Q23"]
    rng = np.random.default_rng(3511)
    one = 1 << 23
    x = np.concatenate([rng.integers(-27 * one, 64 * one, size=20000, dtype=np.int64),
                        rng.integers(-one, one, size=6000, dtype=np.int64),           # k = -1, 0 and 1
                        rng.integers(-64, 64, size=200, dtype=np.int64),
                        np.array([0, 1, -1, 64 * one - 1, 43 * one, 44 * one, -27 * one], np.int64)])
    sig, silu = oracle.sigmoid_q23(x), oracle.silu_q23(x)
    for i, v in enumerate(x.tolist()):
        q = ts_sigmoid_q23(v, table, log2e)
        assert sig[i] == q, v
        assert silu[i] == (v * q) >> 23, v

