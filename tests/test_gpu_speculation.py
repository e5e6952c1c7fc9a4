"""The MFMA GEMM path runs on GUESSED digit counts whenever it has seen its operands before, and relies on the range
tracking inside its kernels plus a guarded recomputation to stay exact.  A variant whose tracking misses one element is
wrong only when a guess is stale, which tests on fresh operands never produce.  Every speculative variant is therefore
driven here with a deliberately stale guess: operands that fit three digits are remembered, ONE element (or the whole
tensor) is then overwritten in place with a wider value, the next call must still match the oracle bit for bit, must
report exactly one guarded recomputation, and the call after it must run on wider digits.  Needs an MI355X."""
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
    kernel.lib.zk_gemm_set_path(2)
    yield kernel
    kernel.lib.zk_gemm_set_path(0)


def host(t):
    return t.cpu().numpy()


class Operand:
    """a host array and its device twin, changed together"""

    def __init__(self, a):
        self.h = np.ascontiguousarray(a)
        self.narrow = self.h.copy()
        self.d = torch.from_numpy(self.h.copy()).cuda()

    def restore(self):
        self.h[...] = self.narrow
        self.d.copy_(torch.from_numpy(self.h))

    def poke(self, index, value):
        self.h[index] = value
        self.d[index] = int(value)


def _stale_guess_rounds(K, call, expect, operands, pokes):
    """call() -> tuple of device outputs, expect() -> tuple of numpy arrays from the operands' host copies (an entry may
    be (rows, array): then only those rows of the flattened-to-2D output are compared); pokes: callables that widen
    something in place"""
    def check(outs, what):
        for o, e in zip(outs, expect()):
            if e is None:
                continue
            if isinstance(e, tuple):
                rows, e = e
                got = host(o).reshape(-1, o.shape[-1])[rows]
            else:
                got = host(o)
            assert np.array_equal(got, e), what

    for n, poke in enumerate(pokes):
        for op in operands:
            op.restore()
        for _ in range(3):          # whatever these addresses were remembered with, the narrow digits are learnt now
            outs = call()
            torch.cuda.synchronize()
        narrow_plan = K.gemm_last_plan()
        assert narrow_plan[0] == 2, "the MFMA path is the one under test"
        check(outs, "narrow operands, poke %d" % n)
        hits = K.lib.zk_gemm_guard_hits()
        poke()
        outs = call()
        assert K.gemm_last_plan() == narrow_plan, "this call is expected to run on the stale guess"
        check(outs, "stale guess, poke %d" % n)
        assert K.lib.zk_gemm_guard_hits() == hits + 1, "poke %d went unnoticed by the range tracking" % n
        outs = call()
        wide_plan = K.gemm_last_plan()
        assert wide_plan[0] == 2 and (wide_plan[1] > narrow_plan[1] or wide_plan[2] > narrow_plan[2]), (narrow_plan, wide_plan)
        check(outs, "relearnt digits, poke %d" % n)
        assert K.lib.zk_gemm_guard_hits() == hits + 1


def _bmm(K, A, W, c, a_rs=1, b_rs=1):
    return lambda: K.int64_bmm_broadcast(A.d, W.d, a_rs, b_rs, c)


WIDE = 1 << 40


@pytest.mark.parametrize("w32", [False, True])
@pytest.mark.parametrize("shape", [(1, 300, 300, 600), (3, 70, 130, 520), (1, 20, 2048, 1100), (1, 130, 96, 200)])
def test_stale_guess_bmm(K, oracle, shape, w32):
    """plain bmm: A from digit planes (four or more tile columns) or split on the fly, int64 and int32 B (the latter
    tracked in 32 bits), several tile rows sharing the tracking of a B tile, split K, 32-row tiles, batches"""
    Bd, M, Kd, N = shape
    rng = np.random.default_rng(sum(shape) + w32)
    A = Operand(rand_i64(rng, (Bd, M, Kd), 20))
    W = Operand(rand_i32(rng, (N, Kd), 16) if w32 else rand_i64(rng, (N, Kd), 16))
    wide_b = (1 << 30) if w32 else -WIDE
    pokes = [lambda: A.poke((Bd - 1, M - 1, Kd - 1), WIDE), lambda: A.poke((0, 0, 0), -WIDE),
             lambda: A.poke((Bd // 2, M // 2, Kd // 3), WIDE), lambda: W.poke((N - 1, Kd - 1), wide_b),
             lambda: W.poke((0, 0), wide_b), lambda: W.poke((N // 2 + 1, Kd // 2 + 3), wide_b),
             lambda: W.poke((N // 3, 33 % Kd), -wide_b - 1 if w32 else WIDE)]
    _stale_guess_rounds(K, _bmm(K, A, W, 29), lambda: oracle.int64_bmm_broadcast(A.h, W.h, 1, 1, 29), [A, W], pokes)


@pytest.mark.parametrize("N", [256, 1024])            # A tracked inside the GEMM kernel / by the plane pre-pass
@pytest.mark.parametrize("side", ["A", "B"])
def test_tracked_digit_counts_at_the_borders(K, oracle, side, N):
    """The kernels track the digit count an operand needs, not its extremes.  n balanced digits hold
    [-0x80..80, 0x7F..7F] (n bytes each): one element exactly on a border must leave the digit count where it is, one
    element past it must raise it by one, on either side of zero, whatever the other elements hold.  The digit count a
    border value ends up with is compared with that of a plain value of the same width."""
    rng = np.random.default_rng(700 + N)
    M, Kd = 64, 256
    keep = []                       # every operand at an address of its own: nothing remembered for it

    def plan_with(value):
        A = rand_i64(rng, (1, M, Kd), 12)
        W = rand_i64(rng, (N, Kd), 12)
        (A if side == "A" else W)[(0, 5, 7) if side == "A" else (N - 3, 9)] = value
        dA, dW = torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda()
        keep.extend((dA, dW))
        for _ in range(3):          # the first call learns the range, the later ones run on it
            C, R = K.int64_bmm_broadcast(dA, dW, 1, 1, 13)
            torch.cuda.synchronize()        # (what a call has seen reaches the next one once its kernels are through)
        Ce, Re = oracle.int64_bmm_broadcast(A, W, 1, 1, 13)
        assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
        return K.gemm_last_plan()
    told_apart = 0
    for n in (2, 3, 4, 5):
        top, bottom = int("7F" * n, 16), -int("80" * n, 16)
        fits, beyond = plan_with(1 << (8 * n - 9)), plan_with(1 << (8 * n - 1))       # n and n + 1 digits for certain
        assert plan_with(top) == fits and plan_with(bottom) == fits, n
        assert plan_with(top + 1) == beyond and plan_with(bottom - 1) == beyond, n
        told_apart += fits != beyond
    # (not every digit count has a kernel of its own: two digits run on three, five on six; some borders must show)
    assert told_apart >= 2


def test_stale_guess_whole_operands_widen(K, oracle):
    """both operands rewritten with full-range values under the same pointers (every tile and every k-step is wide)"""
    rng = np.random.default_rng(5)
    A = Operand(rand_i64(rng, (2, 100, 200), 20))
    W = Operand(rand_i64(rng, (520, 200), 16))

    def widen():
        A.h[...] = rand_i64(rng, A.h.shape, 63)
        W.h[...] = rand_i64(rng, W.h.shape, 63)
        A.d.copy_(torch.from_numpy(A.h))
        W.d.copy_(torch.from_numpy(W.h))
    _stale_guess_rounds(K, _bmm(K, A, W, 7), lambda: oracle.int64_bmm_broadcast(A.h, W.h, 1, 1, 7), [A, W], [widen])


@pytest.mark.parametrize("fallback", ["mfma", "valu"])
@pytest.mark.parametrize("w32", [False, True])
def test_stale_guess_both_kinds_of_guarded_launch(K, oracle, fallback, w32, monkeypatch):
    """the launch behind a speculative product is the widest MFMA instance, one workgroup per compute unit walking the
    tiles (row-major B: nine digits for int64, five for int32), or the vector-ALU tiles (ZK_VALU_FALLBACK, and whatever
    the MFMA form does not take).  Shapes with fewer tiles than compute units and with several tiles per workgroup,
    ragged edges, batches, a remainder or none, every element wide or a single one."""
    import os
    if fallback == "valu":
        monkeypatch.setenv("ZK_VALU_FALLBACK", "1")
    else:
        monkeypatch.delenv("ZK_VALU_FALLBACK", raising=False)
    K.lib.zk_reload_env()
    try:
        rng = np.random.default_rng(900 + w32)
        for Bd, M, Kd, N, c in ((1, 40, 300, 90, 29), (2, 130, 520, 1300, 0), (1, 700, 96, 1500, 33)):
            A = Operand(rand_i64(rng, (Bd, M, Kd), 20))
            W = Operand(rand_i32(rng, (N, Kd), 16) if w32 else rand_i64(rng, (N, Kd), 16))

            def widen():
                A.h[...] = rand_i64(rng, A.h.shape, 63)
                W.h[...] = rand_i32(rng, W.h.shape, 31) if w32 else rand_i64(rng, W.h.shape, 63)
                A.d.copy_(torch.from_numpy(A.h))
                W.d.copy_(torch.from_numpy(W.h))
            # (values of up to five digits make the guarded launch multiply with (5,5), wider ones with nine digits)
            pokes = [widen, lambda: A.poke((Bd - 1, M - 1, Kd - 1), -(1 << 62)), lambda: W.poke((N - 1, 0), (1 << 30) if w32 else (1 << 62)),
                     lambda: A.poke((0, 0, 1), 1 << 37), lambda: W.poke((1, Kd - 1), -(1 << 29) if w32 else -(1 << 36))]
            _stale_guess_rounds(K, _bmm(K, A, W, c), lambda: oracle.int64_bmm_broadcast(A.h, W.h, 1, 1, c), [A, W], pokes)
        # without a remainder
        A = Operand(rand_i64(rng, (1, 70, 200), 20))
        W = Operand(rand_i32(rng, (300, 200), 16) if w32 else rand_i64(rng, (300, 200), 16))
        _stale_guess_rounds(K, lambda: (K.int64_bmm_broadcast(A.d, W.d, 1, 1, 17, want_remainder=False)[0],),
                            lambda: (oracle.int64_bmm_broadcast(A.h, W.h, 1, 1, 17)[0],), [A, W],
                            [lambda: A.poke((0, 3, 5), 1 << 61)])
    finally:
        monkeypatch.delenv("ZK_VALU_FALLBACK", raising=False)
        K.lib.zk_reload_env()


def test_stale_guess_long_k_falls_back_to_the_vector_alu(K, oracle):
    """nine digits over K = 16384 do not fit the int32 accumulators of one pass (the guarded MFMA form does not split K):
    the vector-ALU tiles stand behind such a product"""
    rng = np.random.default_rng(950)
    A = Operand(rand_i64(rng, (1, 40, 16384), 20))
    W = Operand(rand_i64(rng, (70, 16384), 16))
    _stale_guess_rounds(K, _bmm(K, A, W, 29), lambda: oracle.int64_bmm_broadcast(A.h, W.h, 1, 1, 29), [A, W],
                        [lambda: A.poke((0, 39, 16383), -(1 << 62)), lambda: W.poke((5, 7), 1 << 62)])


def test_operands_at_new_addresses_run_on_the_digits_of_their_shape(K, oracle):
    """a product below 2^34 MACs whose operands lie at addresses never seen takes the digits of the last operands of the
    same shapes and does not wait; wider values than those are caught by the guarded launch like any stale guess"""
    rng = np.random.default_rng(960)
    keep = []
    M, Kd, N = 72, 264, 136            # (a shape no other test uses)
    def fresh(bits_a, bits_w):
        a, w = rand_i64(rng, (1, M, Kd), bits_a), rand_i64(rng, (N, Kd), bits_w)
        keep.extend((torch.from_numpy(a).cuda(), torch.from_numpy(w).cuda()))
        C, R = K.int64_bmm_broadcast(keep[-2], keep[-1], 1, 1, 19)
        plan = K.gemm_last_plan()
        Ce, Re = oracle.int64_bmm_broadcast(a, w, 1, 1, 19)
        assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
        torch.cuda.synchronize()
        return plan
    assert fresh(20, 16) == (2, 3, 3)            # first of its shape: sampled
    hits = K.lib.zk_gemm_guard_hits()
    assert fresh(20, 16) == (2, 3, 3)
    assert K.lib.zk_gemm_guard_hits() == hits
    assert fresh(45, 40) == (2, 3, 3)            # runs on the shape's digits, is caught, and teaches the shape
    assert K.lib.zk_gemm_guard_hits() == hits + 1
    plan = fresh(45, 40)
    assert plan[1] >= 6 and plan[2] >= 6 and K.lib.zk_gemm_guard_hits() == hits + 1


def test_stale_guess_fresh_activations_known_weights(K, oracle):
    """what a model does in every layer: a NEW activation tensor against weights seen before.  The digits of A are
    guessed from the activations last multiplied with those weights; wider ones must be caught."""
    rng = np.random.default_rng(11)
    W = Operand(rand_i32(rng, (700, 384), 30))
    keep = []                 # earlier activations stay alive, so every call sees an address it has not seen
    for M in (40, 24):
        Ce = None
        for rep in range(3):
            a = rand_i64(rng, (1, M, 384), 20)
            keep.append(torch.from_numpy(a).cuda())
            C, R = K.int64_bmm_broadcast(keep[-1], W.d, 1, 1, 30)
            Ce, Re = oracle.int64_bmm_broadcast(a, W.h, 1, 1, 30)
            assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
        narrow_plan = K.gemm_last_plan()
        assert narrow_plan[0] == 2 and narrow_plan[1] <= 4
        hits = K.lib.zk_gemm_guard_hits()
        a = rand_i64(rng, (1, M, 384), 20)
        a[0, M - 1, 383] = 1 << 45
        keep.append(torch.from_numpy(a).cuda())
        C, R = K.int64_bmm_broadcast(keep[-1], W.d, 1, 1, 30)
        assert K.gemm_last_plan() == narrow_plan
        Ce, Re = oracle.int64_bmm_broadcast(a, W.h, 1, 1, 30)
        assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
        assert K.lib.zk_gemm_guard_hits() == hits + 1


@pytest.mark.parametrize("rewrite", [False, True])
def test_stale_guess_values_einsum(K, oracle, rewrite):
    """bsht,btc->bshc: an n-contiguous int64 B per batch, read as it lies or through the row-major rewrite"""
    import os
    rng = np.random.default_rng(21 + rewrite)
    Bq, S, H, T, Cc = 2, 9, 8, 200, 300
    P = Operand(rng.integers(0, 1 << 19, size=(Bq, S, H, T), dtype=np.int64))
    V = Operand(rand_i64(rng, (Bq, T, Cc), 20))
    old = os.environ.get("ZK_B_ROWS_MIN_MACS")
    os.environ["ZK_B_ROWS_MIN_MACS"] = "1" if rewrite else "1e30"
    K.lib.zk_reload_env()
    try:
        pokes = [lambda: V.poke((1, T - 1, Cc - 1), WIDE), lambda: V.poke((0, 0, 0), -WIDE), lambda: V.poke((1, 77, 131), WIDE),
                 lambda: P.poke((1, S - 1, H - 1, T - 1), WIDE), lambda: P.poke((0, 2, 3, 5), WIDE)]
        _stale_guess_rounds(K, lambda: (K.einsum_bsht_btc_bshc(P.d, V.d, 23),),
                            lambda: (oracle.einsum_bsht_btc_bshc(P.h, V.h, 23),), [P, V], pokes)
    finally:
        if old is None:
            del os.environ["ZK_B_ROWS_MIN_MACS"]
        else:
            os.environ["ZK_B_ROWS_MIN_MACS"] = old
        K.lib.zk_reload_env()


def test_stale_guess_scores_einsum(K, oracle):
    """bshc,btc->bsht: a k-contiguous B per batch; the wide element sits in the second batch's B"""
    rng = np.random.default_rng(31)
    Bq, S, H, T, Cc = 2, 10, 8, 300, 192
    Q = Operand(rand_i64(rng, (Bq, S, H, Cc), 20))
    Kc = Operand(rand_i64(rng, (Bq, T, Cc), 20))
    pokes = [lambda: Kc.poke((1, T - 1, Cc - 1), WIDE), lambda: Kc.poke((1, 0, 0), -WIDE), lambda: Kc.poke((0, 150, 100), WIDE),
             lambda: Q.poke((1, S - 1, H - 1, Cc - 1), WIDE), lambda: Q.poke((0, 0, 0, 0), -WIDE)]
    _stale_guess_rounds(K, lambda: (K.einsum_bshc_btc_bsht(Q.d, Kc.d, 21),),
                        lambda: (oracle.einsum_bshc_btc_bsht(Q.h, Kc.h, 21),), [Q, Kc], pokes)


def test_stale_guess_per_head_einsums(K, oracle):
    """bshd,hdc->bshc (int32 weights, n-contiguous, one matrix per head) and bshc,hdc->bshd (k-contiguous): the wide
    weight belongs to the last head"""
    rng = np.random.default_rng(41)
    Bq, S, H, D, Cc = 1, 70, 6, 128, 192
    q = Operand(rand_i64(rng, (Bq, S, H, D), 20))
    w1 = Operand(rand_i32(rng, (H, D, Cc), 16))
    pokes = [lambda: w1.poke((H - 1, D - 1, Cc - 1), 1 << 30), lambda: w1.poke((H - 1, 0, 0), -(1 << 30)), lambda: w1.poke((2, 50, 70), 1 << 30),
             lambda: q.poke((0, S - 1, H - 1, D - 1), WIDE), lambda: q.poke((0, 0, 0, 0), WIDE)]
    _stale_guess_rounds(K, lambda: (K.einsum_bshd_hdc_bshc(q.d, w1.d, 30),),
                        lambda: (oracle.einsum_bshd_hdc_bshc(q.h, w1.h, 30),), [q, w1], pokes)
    o = Operand(rand_i64(rng, (Bq, S, H, Cc), 20))
    w2 = Operand(rand_i32(rng, (H, D, Cc), 16))
    pokes = [lambda: w2.poke((H - 1, D - 1, Cc - 1), 1 << 30), lambda: w2.poke((H - 1, 0, 0), -(1 << 30)), lambda: w2.poke((3, 5, 7), 1 << 30),
             lambda: o.poke((0, S - 1, H - 1, Cc - 1), WIDE)]
    _stale_guess_rounds(K, lambda: (K.einsum_bshc_hdc_bshd(o.d, w2.d, 31),),
                        lambda: (oracle.einsum_bshc_hdc_bshd(o.h, w2.h, 31),), [o, w2], pokes)


@pytest.mark.parametrize("M", [20, 200])
def test_stale_guess_prepared_weights(K, oracle, M):
    """B from prepared digit planes (its digit count is exact, nothing of it is tracked): activations that outgrow the
    kernels made for the planes' digit count must be caught, and the next call splits the original weights instead"""
    rng = np.random.default_rng(51 + M)
    A = Operand(rand_i64(rng, (1, M, 512), 20))
    W = Operand(rand_i64(rng, (640, 512), 16))
    K.prepare_weights(W.d)
    try:
        call = _bmm(K, A, W, 29)
        for _ in range(3):          # (the allocator may have handed out an address remembered with wider activations)
            call()
            torch.cuda.synchronize()
        assert K.lib.zk_gemm_last_prepared() == 1
        pokes = [lambda: A.poke((0, M - 1, 511), 1 << 62), lambda: A.poke((0, 0, 0), -(1 << 62)), lambda: A.poke((0, M // 2, 100), 1 << 62)]
        _stale_guess_rounds(K, call, lambda: oracle.int64_bmm_broadcast(A.h, W.h, 1, 1, 29), [A], pokes)
    finally:
        K.release_weights(W.d)


def test_stale_guess_split_tail_tiles_of_a_multi_round_launch(K, oracle):
    """more tiles than compute units: whole tiles in the full rounds, the tiles of the last partial round split along K
    and dealt over the XCDs.  Wide elements in the tail tiles' columns, in the last K slice, and in the planes of A."""
    rng = np.random.default_rng(61)
    M, Kd, N = 512, 1024, 10240
    A = Operand(rand_i64(rng, (1, M, Kd), 20))
    W = Operand(rand_i64(rng, (N, Kd), 16))
    rows = np.array([0, 1, 127, 128, 255, 300, 383, 384, 500, 511])

    def expect():
        Ce, Re = oracle.int64_bmm_broadcast(np.ascontiguousarray(A.h[:, rows]), W.h, 1, 1, 29)
        return (rows, Ce[0]), (rows, Re[0])
    pokes = [lambda: W.poke((N - 1, Kd - 1), WIDE), lambda: W.poke((8192 + 5, 700), -WIDE), lambda: W.poke((9000, 3), WIDE),
             lambda: W.poke((100, 900), WIDE), lambda: A.poke((0, 511, Kd - 1), WIDE), lambda: A.poke((0, 128, 600), -WIDE)]
    _stale_guess_rounds(K, _bmm(K, A, W, 29), expect, [A, W], pokes)


@pytest.mark.parametrize("w32", [False, True])
def test_stale_guess_divided_weights(K, oracle, w32):
    """the head projection's form: B divided by a power of two inside the 32-row kernels, tracked on the divided values"""
    rng = np.random.default_rng(71 + w32)
    M, Kd, N = 24, 2048, 1100
    A = Operand(rand_i64(rng, (1, M, Kd), 20))
    W = Operand(rand_i32(rng, (N, Kd), 24) if w32 else rand_i64(rng, (N, Kd), 24))
    # (an int32 weight divided by 256 needs a fourth digit only at the top of the positive range: three digits hold
    # [-2^23 - 32896, 2^23 - 32896))
    # (the 32-row kernels that divide B stop at five digits: wider operands go to the vector-ALU path)
    wide_b = (1 << 31) - 1 if w32 else (1 << 38) + 12345
    pokes = [lambda: W.poke((N - 1, Kd - 1), wide_b), lambda: W.poke((0, 0), wide_b if w32 else -wide_b), lambda: W.poke((517, 1000), wide_b),
             lambda: A.poke((0, M - 1, Kd - 1), 1 << 28)]
    _stale_guess_rounds(K, _bmm(K, A, W, 29, 1, 256), lambda: oracle.int64_bmm_broadcast(A.h, W.h, 1, 256, 29), [A, W], pokes)


@pytest.mark.parametrize("w32,bits", [(False, (20, 16)), (True, (20, 16)), (True, (28, 28))])
def test_stale_guess_grouped_launch(K, oracle, w32, bits):
    """the routed experts' grouped product: activations gathered into a buffer of their own for every call, weights seen
    before.  Once the weights are known the launch does not wait for its verdict; a guarded launch of the 16-row
    kernels behind it computes everything again when the digits guessed from the last activations (or remembered for
    the weights) were too few.  (28, 28)-bit operands on int32 weights are sixteen digit pairs: the launch that streams the
    weights through LDS rings, whose tiles of at most 16 rows track what they load in their own way."""
    rng = np.random.default_rng(40 + w32 + bits[0])
    T, E, Kr, Kd, N = 150, 10, 4, 192, 520
    idx = np.stack([rng.permutation(E)[:Kr] for _ in range(T)]).astype(np.int64)
    idx[:50, 0] = 3                                  # one expert with more than a tile of rows
    idx[:50, 1:] = np.stack([rng.permutation([0, 1, 2, 4, 5, 6])[: Kr - 1] for _ in range(50)])
    X = Operand(rand_i64(rng, (T, Kd), bits[0]))
    Ws = [Operand(rand_i32(rng, (N, Kd), bits[1]) if w32 else rand_i64(rng, (N, Kd), bits[1])) for _ in range(E)]
    table = K.pointer_table([w.d for w in Ws])
    d = K.moe_dispatch(torch.from_numpy(idx).cuda(), E)
    seg, tok, _ = oracle.moe_dispatch(idx, E)
    busiest = int(np.argmax(np.diff(seg)))
    row_of_busiest = int(tok[seg[busiest] + 40])     # a token in the second tile of the expert with the most rows

    def call():
        xs = K.moe_gather_rows(X.d, d)
        return K.int64_grouped_bmm(xs, table, w32, N, 19, d, want_remainder=True)

    # (four digits where there were three: the 32-row kernels have instances for that; beyond five digits the product
    #  would move to the 16-row kernels altogether)
    wide, wide_w = (1 << 29, 1 << 29) if bits[0] == 20 else (1 << 36, (1 << 31) - 1)       # (a fifth digit where there were four)
    streamed = K.lib.zk_gemm_grouped_streamed_calls()
    pokes = [lambda: X.poke((0, 0), wide), lambda: X.poke((T - 1, Kd - 1), -wide), lambda: X.poke((row_of_busiest, 77), wide),
             lambda: Ws[busiest].poke((N - 1, Kd - 1), -wide_w if bits[0] == 20 else wide_w),      # (no negative int32 needs a fifth digit)
             lambda: Ws[int(idx[T - 1, 0])].poke((0, 0), wide_w)]
    _stale_guess_rounds(K, call, lambda: oracle.grouped_bmm(X.h[tok], [w.h for w in Ws], seg, 19), [X] + Ws, pokes)
    if bits[0] == 28:
        assert K.lib.zk_gemm_grouped_streamed_calls() - streamed >= 5 * 4, "the launches under test were to run on the streamed kernel"


def test_declined_product_runs_although_an_older_error_is_pending(K, oracle):
    """the error channel keeps the first error until it is cleared; a later product that the MFMA path merely declines
    (an operand divisor on A) must still run on the other path, whatever that channel holds"""
    rng = np.random.default_rng(81)
    A = rand_i64(rng, (1, 50, 200), 30)
    W = rand_i64(rng, (70, 200), 30)
    dA, dW = torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda()
    C = torch.zeros((1, 50, 70), dtype=torch.int64, device="cuda")
    R = torch.zeros_like(C)
    K.lib.zk_gemm_set_path(0)
    K.lib.zk_gemm_set_path(7)                      # a bad argument: recorded, never cleared by the caller
    assert K.lib.zk_last_error() == 1
    try:
        K.lib.int64_64_bmm_broadcast_launcher(dA.data_ptr(), dW.data_ptr(), C.data_ptr(), R.data_ptr(), 2, 1, 13, 1, 50, 200, 70)
        Ce, Re = oracle.int64_bmm_broadcast(A, W, 2, 1, 13)
        assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
        assert K.lib.zk_last_error() == 1          # still the old error
    finally:
        K.lib.zk_clear_error()
        K.lib.zk_gemm_set_path(2)


def test_workspace_is_reported_and_released(K, oracle):
    """the scratch the library keeps between calls can be seen and returned; the next call allocates it again"""
    rng = np.random.default_rng(91)
    A = rand_i64(rng, (1, 200, 512), 20)
    W = rand_i64(rng, (640, 512), 16)
    dA, dW = torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda()
    Ce, Re = oracle.int64_bmm_broadcast(A, W, 1, 1, 29)
    C, R = K.int64_bmm_broadcast(dA, dW, 1, 1, 29)
    assert np.array_equal(host(C), Ce)
    scratch, prepared = K.workspace_bytes()
    assert scratch > 0
    K.prepare_weights(dW)
    assert K.workspace_bytes()[1] >= prepared + 640 * 512 * 3
    K.release_weights(dW)
    assert K.workspace_bytes()[1] == prepared
    K.release_workspace()
    assert K.workspace_bytes()[0] < scratch
    C, R = K.int64_bmm_broadcast(dA, dW, 1, 1, 29)
    assert np.array_equal(host(C), Ce) and np.array_equal(host(R), Re)
