"""ctypes front end of the CPU oracle (libzkoracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product (the HIP library and its `kernel`
module) never imports this file.

All functions take and return C-contiguous numpy arrays and mirror the Python
operator API of the reference's inference/kernel.py:341-688 (same argument
order and meaning), except that nothing lives on a GPU.

Functions below that are compositions in numpy (the fusions, the MoE path, the checkpoint quantisation) restate
tensor ops of inference/model.py and inference/convert2.py, cited where they are defined.  Parity unpinned (the
reference leaves them to its device, and nothing it ships can confirm the choice made here): float values outside
the integer range and NaN in the checkpoint quantisation (fixed as saturation and 0); see zk_oracle.c for the
integer kernels' list.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# ZK_ORACLE_LIB names another build of zk_oracle.c to load instead: the mutant test uses it to show that the pin
# suite rejects perturbed copies of the oracle
_SO = os.environ.get("ZK_ORACLE_LIB") or os.path.join(_HERE, "libzkoracle.so")


def build(force=False):
    """Compile libzkoracle.so with gcc (a second or two)."""
    src = os.path.join(_HERE, "zk_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libzkoracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


def _load():
    if not os.path.exists(_SO):
        build()
    lib = ctypes.CDLL(_SO)
    vp, ll, ci, cl = ctypes.c_void_p, ctypes.c_longlong, ctypes.c_int, ctypes.c_long
    for name in ("ora_int64_64_bmm_broadcast", "ora_int64_32_bmm_broadcast"):
        getattr(lib, name).argtypes = [vp, vp, vp, vp, ll, ll, ll, ci, ci, ci, ci]
    for name in ("ora_einsum_bshd_hdc_bshc", "ora_einsum_bshc_btc_bsht",
                 "ora_einsum_bsht_btc_bshc", "ora_einsum_bshc_hdc_bshd"):
        getattr(lib, name).argtypes = [vp, vp, vp, ll, ci, ci, ci, ci, ci]
    lib.ora_complex_int64_mul.argtypes = [vp, vp, vp, ci, ci, ci, ci]
    lib.ora_rms_stat.argtypes = [vp, vp, ci, ci, ll, ll]
    lib.ora_rms_stat.restype = ci
    lib.ora_rms_norm_32.argtypes = [vp, vp, vp, vp, ci, ci]
    lib.ora_rms_norm_64.argtypes = [vp, vp, vp, vp, ci, ci]
    for name in ("ora_softmax_init_q19", "ora_softmax_init_q21", "ora_silu_init_q23", "ora_silu_init_q25"):
        getattr(lib, name).argtypes = [vp]
    for name in ("ora_softmax_q19", "ora_softmax_q21"):
        getattr(lib, name).argtypes = [vp, vp, vp, vp, ci, ci, ci, ci]
    for name in ("ora_act_q23", "ora_act_q25"):
        getattr(lib, name).argtypes = [vp, vp, vp, cl, ci]
    lib.ora_bf16_to_int32.argtypes = [vp, vp, cl, ci, ci]
    lib.ora_float32_to_int64.argtypes = [vp, vp, cl, ci]
    lib.ora_gate_route.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci]
    lib.ora_set_threads.argtypes = [ci]
    lib.ora_max_threads.restype = ci
    return lib


_lib = _load()


def set_threads(n):
    _lib.ora_set_threads(int(n))


def max_threads():
    return int(_lib.ora_max_threads())


def _c(a, dtype=np.int64):
    a = np.ascontiguousarray(a)
    assert a.dtype == dtype, (a.dtype, dtype)
    return a


def _p(a):
    return a.ctypes.data


def int64_bmm_broadcast(A, B, a_rescale, b_rescale, c_rescale):
    """(C, R) of inference/kernel.py:341-371."""
    A = _c(A)
    Bdim, M, K = A.shape
    N, K2 = B.shape
    assert K2 == K
    C = np.empty((Bdim, M, N), np.int64)
    R = np.empty((Bdim, M, N), np.int64)
    if B.dtype == np.int64:
        B = _c(B)
        _lib.ora_int64_64_bmm_broadcast(_p(A), _p(B), _p(C), _p(R), a_rescale, b_rescale, c_rescale, Bdim, M, K, N)
    else:
        B = _c(B, np.int32)
        _lib.ora_int64_32_bmm_broadcast(_p(A), _p(B), _p(C), _p(R), a_rescale, b_rescale, c_rescale, Bdim, M, K, N)
    return C, R


def einsum_bshd_hdc_bshc(A, B, rescale):
    A, B = _c(A), _c(B, np.int32)
    Bt, S, H, D = A.shape
    assert B.shape[0] == H and B.shape[1] == D
    Cp = B.shape[2]
    out = np.empty((Bt, S, H, Cp), np.int64)
    _lib.ora_einsum_bshd_hdc_bshc(_p(A), _p(B), _p(out), rescale, Bt, S, H, D, Cp)
    return out


def einsum_bshc_btc_bsht(A, B, rescale):
    A, B = _c(A), _c(B)
    Bsz, S, H, Cdim = A.shape
    T = B.shape[1]
    assert B.shape[0] == Bsz and B.shape[2] == Cdim
    out = np.empty((Bsz, S, H, T), np.int64)
    _lib.ora_einsum_bshc_btc_bsht(_p(A), _p(B), _p(out), rescale, Bsz, S, H, T, Cdim)
    return out


def einsum_bsht_btc_bshc(A, B, rescale):
    A, B = _c(A), _c(B)
    Bsz, S, H, T = A.shape
    Cdim = B.shape[2]
    assert B.shape[0] == Bsz and B.shape[1] == T
    out = np.empty((Bsz, S, H, Cdim), np.int64)
    _lib.ora_einsum_bsht_btc_bshc(_p(A), _p(B), _p(out), rescale, Bsz, S, H, T, Cdim)
    return out


def einsum_bshc_hdc_bshd(A, B, rescale):
    A, B = _c(A), _c(B, np.int32)
    Bsz, S, H, Cdim = A.shape
    D = B.shape[1]
    assert B.shape[0] == H and B.shape[2] == Cdim
    out = np.empty((Bsz, S, H, D), np.int64)
    _lib.ora_einsum_bshc_hdc_bshd(_p(A), _p(B), _p(out), rescale, Bsz, S, H, D, Cdim)
    return out


def complex_int64_mul_broadcast(A, B):
    """A [B,S,H,D,2], B [1,S,1,D,2] (inference/kernel.py:373-395; headDim = A.shape[3])."""
    A, B = _c(A), _c(B)
    out = np.empty_like(A)
    _lib.ora_complex_int64_mul(_p(A), _p(B), _p(out), A.shape[0], A.shape[1], A.shape[2], A.shape[3])
    return out


def rms_stat(A, eps, dim):
    A = _c(A)
    M, N = A.shape
    rms = np.empty((M,), np.int64)
    rc = _lib.ora_rms_stat(_p(A), _p(rms), M, N, eps, dim)
    assert rc == 0, "(eps + sum a^2)//dim does not fit 128 bits"
    return rms


def rms_norm_apply(A, W, rms):
    A, rms = _c(A), _c(rms)
    M, N = A.shape
    C = np.empty((M, N), np.int64)
    if W.dtype == np.int32:
        W = _c(W, np.int32)
        _lib.ora_rms_norm_32(_p(A), _p(W), _p(rms), _p(C), M, N)
    else:
        W = _c(W)
        _lib.ora_rms_norm_64(_p(A), _p(W), _p(rms), _p(C), M, N)
    return C


def RMS_Norm_int64(A, W, eps, dim):
    """(C, rms[:M]) of inference/kernel.py:528-550 (the reference returns its whole 500-row buffer)."""
    rms = rms_stat(A, eps, dim)
    return rms_norm_apply(A, W, rms), rms


def RMS_Norm_residual_int64(X, Y, k, W, eps, dim):
    """(X', C, rms) for X' = X + Y * 2^k in wrapping int64 (torch's tensor ops at inference/model.py:1465, 1472)
    followed by the norm of inference/model.py:1468 / the next block's :1453."""
    Xn = (_c(X).view(np.uint64) + (_c(Y).view(np.uint64) << np.uint64(k))).view(np.int64)
    C, rms = RMS_Norm_int64(Xn, W, eps, dim)
    return Xn, C, rms


def _lut(fn):
    lut = np.zeros((256,), np.int64)
    fn(_p(lut))
    return lut


def softmax_init_q19():
    return _lut(_lib.ora_softmax_init_q19)


def softmax_init_q21():
    return _lut(_lib.ora_softmax_init_q21)


def silu_init_q23():
    return _lut(_lib.ora_silu_init_q23)


def silu_init_q25():
    return _lut(_lib.ora_silu_init_q25)


def _softmax(fn, R, lut):
    R = _c(R)
    Bsz, S, H, T = R.shape
    C = np.empty_like(R)
    W = np.empty_like(R)
    fn(_p(R), _p(C), _p(W), _p(_c(lut)), Bsz, S, H, T)
    return C, W


def softmax_q19(R, lut=None):
    """Returns (C, w): the probabilities and the weights the reference leaves in its input buffer."""
    return _softmax(_lib.ora_softmax_q19, R, softmax_init_q19() if lut is None else lut)


def softmax_q21(R, lut=None):
    return _softmax(_lib.ora_softmax_q21, R, softmax_init_q21() if lut is None else lut)


def _act(fn, R, lut, mode):
    R = _c(R)
    C = np.empty_like(R)
    fn(_p(R), _p(C), _p(_c(lut)), R.size, mode)
    return C


def silu_q23(R, lut=None):
    return _act(_lib.ora_act_q23, R, silu_init_q23() if lut is None else lut, 0)


def sigmoid_q23(R, lut=None):
    return _act(_lib.ora_act_q23, R, silu_init_q23() if lut is None else lut, 1)


def silu_q25(R, lut=None):
    return _act(_lib.ora_act_q25, R, silu_init_q25() if lut is None else lut, 0)


def sigmoid_q25(R, lut=None):
    return _act(_lib.ora_act_q25, R, silu_init_q25() if lut is None else lut, 1)


def softmax_q19_scores(s1, s2, mask, mul=94, div=695, lut=None):
    """(scores, C) of the fused call: the tensor ops of inference/model.py:896-906 restated with numpy's wrapping int64
    arithmetic and floor division (what torch's `*`, `+` and `//` do), then softmax_q19 (:908-915)."""
    with np.errstate(over="ignore"):
        x = _c(s1).copy()
        if s2 is not None:
            x = x + _c(s2)
        x = (x * np.int64(mul)) // np.int64(div)
        if mask is not None:
            x = x + _c(mask)[None, :, None, :]
    return x, softmax_q19(x, lut)[0]


def silu_mul_q23(R, U, lut=None):
    """(silu, C) of the fused call: silu_q23, then the wrapping product and the floor shift of inference/model.py:1048"""
    s = silu_q23(R, lut)
    with np.errstate(over="ignore"):
        return s, (s * _c(U)) >> 23


def gate_route(scores, bias, n_groups, topk_groups, topk):
    """(weights, indices, raw_weights) of Gate.forward's routing (inference/model.py:1143-1208); scores [T,E] int64,
    bias [E] int32 or None"""
    scores = _c(scores)
    T, E = scores.shape
    assert E <= 1024 and n_groups <= 64 and E % n_groups == 0
    w = np.empty((T, topk), np.int64)
    idx = np.empty((T, topk), np.int64)
    raw = np.empty((T, topk), np.int64)
    b = None if bias is None else _c(bias, np.int32)
    _lib.ora_gate_route(_p(scores), None if b is None else _p(b), _p(w), _p(idx), _p(raw), T, E, n_groups, topk_groups, topk)
    return w, idx, raw


def moe_dispatch(indices, n_experts):
    """(seg [E+1], sorted_token [T*K], sorted_pos [T,K]): the (token, slot) entries sorted by expert, stably, so an
    expert sees its tokens in ascending order (what torch.where gives MoE.forward, inference/model.py:1357-1365)"""
    T, K = indices.shape
    flat = np.asarray(indices).ravel()
    order = np.argsort(flat, kind="stable")
    seg = np.concatenate([[0], np.cumsum(np.bincount(flat, minlength=n_experts))]).astype(np.int32)
    pos = np.empty(T * K, np.int32)
    pos[order] = np.arange(T * K, dtype=np.int32)
    return seg, (order // K).astype(np.int32), pos.reshape(T, K)


def grouped_bmm(A_sorted, weights_list, seg, c_rescale):
    """(C, R) [rows,N]: int64_bmm_broadcast of every expert's segment of rows with that expert's matrix"""
    N = weights_list[0].shape[0]
    C = np.zeros((A_sorted.shape[0], N), np.int64)
    R = np.zeros_like(C)
    for e, w in enumerate(weights_list):
        r0, r1 = int(seg[e]), int(seg[e + 1])
        if r1 > r0:
            c, r = int64_bmm_broadcast(np.ascontiguousarray(A_sorted[None, r0:r1]), w, 1, 1, c_rescale)
            C[r0:r1], R[r0:r1] = c[0], r[0]
    return C, R


def moe_experts(x, weights, indices, w1, w3, w2, c13, c2):
    """The routed experts of MoE.forward as the reference loops over them (inference/model.py:1355-1381): for every
    expert with tokens, Expert_int.forward on those tokens (:1247-1281), times the routing weight, floor-divided by
    2^23 and added to the tokens' rows."""
    T, dim = x.shape
    y = np.zeros((T, dim), np.int64)
    for e in range(len(w1)):
        tok, slot = np.nonzero(np.asarray(indices) == e)
        if tok.size == 0:
            continue
        xe = np.ascontiguousarray(x[tok])[None]
        r1, _ = int64_bmm_broadcast(xe, w1[e], 1, 1, c13)
        r2, _ = int64_bmm_broadcast(xe, w3[e], 1, 1, c13)
        _, h = silu_mul_q23(r1, r2)
        ye, _ = int64_bmm_broadcast(h, w2[e], 1, 1, c2)
        with np.errstate(over="ignore"):
            np.add.at(y, tok, (ye[0] * weights[tok, slot][:, None]) >> 23)
    return y


def bf16_to_int32_2d(bits, rescale):
    """bits: uint16 bf16 patterns [rows, cols] -> int32 fixed point (inference/int64_gemm.cu:92-132)"""
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, np.int32)
    _lib.ora_bf16_to_int32(_p(bits), _p(out), bits.size, rescale, 0)
    return out


def wkv_b_bf16_to_int32(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, np.int32)
    _lib.ora_bf16_to_int32(_p(bits), _p(out), bits.size, 25, 1)
    return out


def _e4m3fn_table():
    """the 256 values of an OCP e4m3fn byte as float32: 1 sign, 4 exponent (bias 7), 3 mantissa bits; no infinities,
    S.1111.111 is NaN"""
    t = np.empty(256, np.float32)
    for b in range(256):
        e, m = (b >> 3) & 15, b & 7
        if e == 15 and m == 7:
            v = float("nan")
        elif e == 0:
            v = m * 2.0 ** -9
        else:
            v = (1 + m / 8.0) * 2.0 ** (e - 7)
        t[b] = -v if b & 0x80 else v
    return t


def _round_to_bf16(x):
    """float32 array -> nearest bfloat16 (ties to even), returned as float32"""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    r = np.where(np.isnan(x), np.uint32(0x7FC00000), r).astype(np.uint32)
    return r.view(np.float32)


def _round_to_int(z, dtype):
    """round half to even, then the float -> integer conversion of the reference's device: saturating, NaN -> 0"""
    info = np.iinfo(dtype)
    r = np.rint(z.astype(np.float64))
    out = np.zeros(z.shape, dtype)
    ok = ~np.isnan(r)
    hi, lo = r >= float(info.max) + 1.0, r <= float(info.min)
    mid = ok & ~hi & ~lo
    out[mid] = r[mid].astype(dtype)
    out[ok & hi] = info.max
    out[ok & lo] = info.min
    return out


def fp8_block_scaled_to_int32(w_bytes, scale, k, block=128):
    """(weight_dequant(w, scale).to(float32) * 2**k).round().to(int32): inference/convert2.py:144-147 with the Triton
    kernel of inference/kernel.py:67-117 (x.to(float32) * s, stored as bfloat16) restated operation by operation."""
    w_bytes = np.ascontiguousarray(w_bytes, np.uint8)
    rows, cols = w_bytes.shape
    s = np.repeat(np.repeat(np.ascontiguousarray(scale, np.float32), block, axis=0), block, axis=1)[:rows, :cols]
    with np.errstate(over="ignore", invalid="ignore"):
        y = _round_to_bf16(_e4m3fn_table()[w_bytes] * s)             # float32 multiply, then bfloat16 store
        z = y * np.float32(2.0 ** k)                                 # exact unless it overflows to infinity
    return _round_to_int(z, np.int32)


def bf16_scaled_round(bits, k, dtype):
    """(p.to(float32) * 2**k).round().to(dtype) for bfloat16 bit patterns (inference/convert2.py:250-262, 290-295)"""
    x = (np.ascontiguousarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        z = x * np.float32(2.0 ** k)
    return _round_to_int(z, dtype)


def float32_to_int64_2d(bits, rescale):
    bits = _c(bits, np.uint32)
    out = np.empty(bits.shape, np.int64)
    _lib.ora_float32_to_int64(_p(bits), _p(out), bits.size, rescale)
    return out
