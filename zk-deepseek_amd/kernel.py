"""Python operator API over libint64gemm.so for AMD MI355X.

Same module name, function names, argument order and return values as the reference's
inference/kernel.py:341-688, so `from kernel import ...` in the reference's model.py
(inference/model.py:13-15) resolves against this file unchanged.  PyTorch is used only to
allocate outputs and hand device pointers to the C ABI (include/int64gemm.h).

Differences from the reference, all deliberate:
  * the RMS statistic is computed on the device (one launch) instead of one `.item()` sync per
    element (inference/kernel.py:477-494, 539-542);
  * every call checks the library's error channel and raises RuntimeError instead of returning
    uninitialised tensors;
  * `act_quant`, `weight_dequant`, `fp8_gemm` (Triton fp8 leftovers that no int64 layer reaches) are
    importable names that raise NotImplementedError.
There is no CPU fallback: if the shared object is missing, importing this module raises.
"""
import atexit
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))


def _find_library():
    # the reference loads "./libint64gemm.so" relative to the working directory (inference/kernel.py:206)
    for cand in (os.path.join(os.getcwd(), "libint64gemm.so"), os.path.join(_HERE, "libint64gemm.so")):
        if os.path.exists(cand):
            return cand
    raise ImportError(
        "libint64gemm.so not found in the working directory or next to kernel.py; "
        "build it with `python zk-deepseek_amd/build.py` (hipcc, gfx950). There is no CPU fallback.")


LIB_PATH = _find_library()
lib = ctypes.CDLL(LIB_PATH)

_vp, _ll, _ci = ctypes.c_void_p, ctypes.c_longlong, ctypes.c_int

lib.int64_64_bmm_broadcast_launcher.argtypes = [_vp, _vp, _vp, _vp, _ll, _ll, _ll, _ci, _ci, _ci, _ci]
lib.int64_32_bmm_broadcast_launcher.argtypes = [_vp, _vp, _vp, _vp, _ll, _ll, _ll, _ci, _ci, _ci, _ci]
lib.complex_int64_mul.argtypes = [_vp, _vp, _vp, _ci, _ci, _ci, _ci]
lib.rms_norm_32.argtypes = [_vp, _vp, _vp, _vp, _ci, _ci]
lib.rms_norm_64.argtypes = [_vp, _vp, _vp, _vp, _ci, _ci]
for _n in ("einsum_bshd_hdc_bshc", "einsum_bshc_btc_bsht", "einsum_bsht_btc_bshc", "einsum_bshc_hdc_bshd"):
    getattr(lib, _n).argtypes = [_vp, _vp, _vp, _ll, _ci, _ci, _ci, _ci, _ci]
lib.softmax_q21.argtypes = [_vp, _vp, _vp, _ci, _ci, _ci, _ci]
lib.softmax_q19.argtypes = [_vp, _vp, _vp, _ci, _ci, _ci, _ci]
for _n in ("softmax_init_q21", "softmax_init_q19", "silu_init_q25", "silu_init_q23"):
    getattr(lib, _n).argtypes = [_vp]
for _n in ("silu_q25", "sigmoid_q25", "silu_q23", "sigmoid_q23"):
    getattr(lib, _n).argtypes = [_vp, _vp, _vp, _ci, _ci, _ci]
for _n in ("bf16_to_int32_2d", "float32_to_int64_2d"):
    getattr(lib, _n).argtypes = [_vp, _vp, _ci, _ci, _ci]
lib.wkv_b_bf16_to_int32.argtypes = [_vp, _vp, _ci, _ci]
lib.fp8_block_scaled_to_int32.argtypes = [_vp, _vp, _vp, _ci, _ci, _ci]
lib.bf16_scaled_round_to_int32.argtypes = [_vp, _vp, ctypes.c_long, _ci]
lib.bf16_scaled_round_to_int64.argtypes = [_vp, _vp, ctypes.c_long, _ci]
lib.zk_gemm_prepare_weights.argtypes = [_vp, _ci, _ci, _ci, _ci]
lib.zk_gemm_release_weights.argtypes = [_vp]
# additions without a reference counterpart
lib.rms_stat_int64.argtypes = [_vp, _vp, _ci, _ci, _ll, _ll]
lib.rms_norm_fused_32.argtypes = [_vp, _vp, _vp, _vp, _ci, _ci, _ll, _ll]
lib.rms_norm_fused_64.argtypes = [_vp, _vp, _vp, _vp, _ci, _ci, _ll, _ll]
lib.rms_norm_residual_fused_32.argtypes = [_vp, _vp, _ci, _vp, _vp, _vp, _vp, _ci, _ci, _ll, _ll]
lib.rms_norm_residual_fused_64.argtypes = [_vp, _vp, _ci, _vp, _vp, _vp, _vp, _ci, _ci, _ll, _ll]
lib.zk_last_error.restype = _ci
lib.zk_last_error_string.restype = ctypes.c_char_p
lib.zk_softmax_clobber_input.argtypes = [_ci]
lib.zk_gemm_set_path.argtypes = [_ci]
lib.zk_gemm_get_path.restype = _ci
lib.zk_gemm_last_plan.argtypes = [ctypes.POINTER(_ci), ctypes.POINTER(_ci), ctypes.POINTER(_ci)]
lib.zk_timer_stop_ms.restype = ctypes.c_float
lib.zk_gemm_guard_hits.restype = ctypes.c_long
lib.zk_gemm_last_pairs.restype = ctypes.c_int
lib.zk_gemm_grouped_mfma_calls.restype = ctypes.c_long
lib.zk_gemm_grouped_streamed_calls.restype = ctypes.c_long
lib.zk_gemm_pipe_calls.restype = ctypes.c_long
lib.softmax_q19_scores.argtypes = [_vp] * 6 + [_ci] * 4 + [ctypes.c_longlong] * 2
lib.silu_mul_q23.argtypes = [_vp] * 5 + [_ci] * 3
lib.gate_route_q23.argtypes = [_vp] * 5 + [_ci] * 5
lib.gate_sigmoid_route_q23.argtypes = [_vp] * 7 + [_ci] * 5
lib.moe_dispatch.argtypes = [_vp, _ci, _ci, _ci] + [_vp] * 6
lib.moe_gather_rows.argtypes = [_vp, _vp, _vp, _ci, _ci]
lib.int64_grouped_bmm_launcher.argtypes = [_vp, _vp, _ci, _vp, _vp, ctypes.c_longlong, _vp, _vp, _vp, _ci, _ci, _ci, _ci]
lib.moe_combine.argtypes = [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci]
lib.zk_dump_device.argtypes = [ctypes.c_char_p, _vp, ctypes.c_size_t]
lib.zk_dump_host.argtypes = [ctypes.c_char_p, _vp, ctypes.c_size_t]
lib.zk_dump_flush.restype = ctypes.c_long
lib.zk_probe_mfma_i8_tops.argtypes = [_ci, _ci, _ci]
lib.zk_probe_mfma_i8_tops.restype = ctypes.c_double
lib.zk_probe_launch_pair_us.argtypes = [_ci, _ci]
lib.zk_probe_launch_pair_us.restype = ctypes.c_double
lib.zk_probe_store_gbps.argtypes = [ctypes.c_long, _ci]
lib.zk_probe_store_gbps.restype = ctypes.c_double
lib.zk_workspace_bytes.restype = ctypes.c_size_t
lib.zk_prepared_weights_bytes.restype = ctypes.c_size_t


def _check(what):
    code = lib.zk_last_error()
    if code != 0:
        msg = lib.zk_last_error_string().decode()
        lib.zk_clear_error()
        raise RuntimeError("%s failed (code %d): %s" % (what, code, msg))


# Prepared planes are found by the address of the weights, and nothing of B is read or checked on that path: were the
# tensor freed, torch's allocator could hand its address to another weight matrix of the same shape, which would then be
# multiplied with the old planes.  So the tensors (for a pointer table: the table and, when given, the matrices it points
# at) are kept alive here until release_weights.
_prepared_keepalive = {}


def prepare_weights(W, groups=0, N=None, K=None, b32=False, matrices=None):
    """Split a weight matrix [N,K] (int64 or int32) or, with groups > 0, every matrix of the device pointer table `W` made
    by pointer_table (b32 says whether they are int32; pass the tensors themselves as `matrices` so that they are kept
    alive too) into digit planes once; later int64_bmm_broadcast / int64_grouped_bmm calls with the same tensor read the
    planes instead of splitting the weights in every tile.  The weights must not change until release_weights."""
    assert W.is_cuda and W.is_contiguous()
    if groups == 0:
        assert W.dim() == 2 and W.dtype in (torch.int64, torch.int32)
        N, K = W.shape
        b32 = W.dtype == torch.int32
    else:
        assert W.dtype == torch.int64 and W.numel() == groups
    if lib.zk_gemm_prepare_weights(W.data_ptr(), 1 if b32 else 0, int(groups), int(N), int(K)) != 0:
        _check("prepare_weights")
    _prepared_keepalive[W.data_ptr()] = (W, matrices)


def release_weights(W):
    lib.zk_gemm_release_weights(W.data_ptr())
    _prepared_keepalive.pop(W.data_ptr(), None)


def workspace_bytes():
    """(scratch bytes, bytes of prepared digit planes) the library holds on the device right now"""
    return int(lib.zk_workspace_bytes()), int(lib.zk_prepared_weights_bytes())


def release_workspace():
    """waits for the device and frees the library's scratch buffers (they are allocated again on demand)"""
    lib.zk_release_workspace()


def gemm_last_pairs():
    """i8 digit products per int64 multiply-add in the last GEMM-like call (0 on the VALU path)"""
    return int(lib.zk_gemm_last_pairs())


def gemm_last_plan():
    """(path, limbs_a, limbs_b) of the last GEMM-shaped call: path 1 = VALU, 2 = i8 MFMA."""
    p, a, b = _ci(), _ci(), _ci()
    lib.zk_gemm_last_plan(ctypes.byref(p), ctypes.byref(a), ctypes.byref(b))
    return p.value, a.value, b.value


def act_quant(*args, **kwargs):
    raise NotImplementedError("act_quant belongs to the fp8 path, which the int64 model never reaches")


def weight_dequant(*args, **kwargs):
    raise NotImplementedError("weight_dequant belongs to the offline fp8 checkpoint converter")


def fp8_gemm(*args, **kwargs):
    raise NotImplementedError("fp8_gemm belongs to the fp8 path, which the int64 model never reaches")


def int64_bmm_broadcast(A: torch.Tensor, B: torch.Tensor, a_rescale, b_rescale, c_rescale, want_remainder=True):
    """(B, M, K) x (N, K) -> quotient C and remainder R, both (B, M, N) int64.
    want_remainder=False (not in the reference) skips the remainder's store and returns (C, None)."""
    assert A.dtype == torch.int64
    assert A.is_cuda and B.is_cuda
    Bdim, M, K = A.shape
    N, K2 = B.shape
    assert K2 == K

    C = torch.empty((Bdim, M, N), dtype=torch.int64, device=A.device)
    R = torch.empty((Bdim, M, N), dtype=torch.int64, device=A.device) if want_remainder else None
    r_ptr = R.data_ptr() if want_remainder else None

    if B.dtype == torch.int64:
        lib.int64_64_bmm_broadcast_launcher(A.data_ptr(), B.data_ptr(), C.data_ptr(), r_ptr,
                                            a_rescale, b_rescale, c_rescale, Bdim, M, K, N)
    elif B.dtype == torch.int32:
        lib.int64_32_bmm_broadcast_launcher(A.data_ptr(), B.data_ptr(), C.data_ptr(), r_ptr,
                                            a_rescale, b_rescale, c_rescale, Bdim, M, K, N)
    else:
        raise TypeError(f"Unsupported B type: {B.dtype}")
    _check("int64_bmm_broadcast")
    return (C, R)


def complex_int64_mul_broadcast(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """Complex multiply in Q42; A [batch, seq, heads, headDim, 2], B [1, seq, 1, headDim, 2]."""
    assert A.dtype == torch.int64 and B.dtype == torch.int64
    assert A.is_cuda and B.is_cuda
    batch, seqLen, head, headDim = A.shape[0], A.shape[1], A.shape[2], A.shape[3]
    C = torch.empty(A.shape, dtype=torch.int64, device=A.device)
    lib.complex_int64_mul(A.data_ptr(), B.data_ptr(), C.data_ptr(), batch, seqLen, head, headDim)
    _check("complex_int64_mul_broadcast")
    return C


def einsum_bshd_hdc_bshc(A: torch.Tensor, B: torch.Tensor, rescale) -> torch.Tensor:
    assert A.shape[2] == B.shape[0] and A.shape[3] == B.shape[1]
    assert A.is_cuda and B.is_cuda
    assert A.dtype == torch.int64 and B.dtype == torch.int32
    Batch, S, H, D = A.shape
    Cp = B.shape[2]
    C = torch.empty([Batch, S, H, Cp], dtype=torch.int64, device=A.device)
    lib.einsum_bshd_hdc_bshc(A.data_ptr(), B.data_ptr(), C.data_ptr(), rescale, Batch, S, H, D, Cp)
    _check("einsum_bshd_hdc_bshc")
    return C


def einsum_bshc_btc_bsht(A: torch.Tensor, B: torch.Tensor, rescale) -> torch.Tensor:
    Bsz, S, H, Cdim = A.shape
    T = B.shape[1]
    assert Bsz == B.shape[0] and Cdim == B.shape[2]
    assert A.is_cuda and B.is_cuda
    assert A.dtype == torch.int64 and B.dtype == torch.int64
    C = torch.empty([Bsz, S, H, T], dtype=torch.int64, device=A.device)
    lib.einsum_bshc_btc_bsht(A.data_ptr(), B.data_ptr(), C.data_ptr(), rescale, Bsz, S, H, T, Cdim)
    _check("einsum_bshc_btc_bsht")
    return C


def einsum_bsht_btc_bshc(A: torch.Tensor, B: torch.Tensor, rescale) -> torch.Tensor:
    Bsz, S, H, T = A.shape
    Cdim = B.shape[2]
    assert Bsz == B.shape[0] and T == B.shape[1]
    assert A.is_cuda and B.is_cuda
    assert A.dtype == torch.int64 and B.dtype == torch.int64
    C = torch.empty([Bsz, S, H, Cdim], dtype=torch.int64, device=A.device)
    lib.einsum_bsht_btc_bshc(A.data_ptr(), B.data_ptr(), C.data_ptr(), rescale, Bsz, S, H, T, Cdim)
    _check("einsum_bsht_btc_bshc")
    return C


def einsum_bshc_hdc_bshd(A: torch.Tensor, B: torch.Tensor, rescale) -> torch.Tensor:
    Bsz, S, H, Cdim = A.shape
    D = B.shape[1]
    assert H == B.shape[0] and Cdim == B.shape[2]
    assert A.is_cuda and B.is_cuda
    assert A.dtype == torch.int64 and B.dtype == torch.int32
    C = torch.empty([Bsz, S, H, D], dtype=torch.int64, device=A.device)
    lib.einsum_bshc_hdc_bshd(A.data_ptr(), B.data_ptr(), C.data_ptr(), rescale, Bsz, S, H, D, Cdim)
    _check("einsum_bshc_hdc_bshd")
    return C


def int64_RMS0(A: torch.Tensor, eps: int, dim: int) -> int:
    """isqrt((eps + sum a^2) // dim) of a 1-D int64 tensor, as a Python int."""
    assert A.dtype == torch.int64
    assert A.ndim == 1
    assert A.is_cuda
    out = torch.empty((1,), dtype=torch.int64, device=A.device)
    A = A.contiguous()
    lib.rms_stat_int64(A.data_ptr(), out.data_ptr(), 1, A.shape[0], eps, dim)
    _check("int64_RMS0")
    return int(out.item())


# The reference keeps one 500-row host buffer and returns it whole (rows >= M keep older values);
# callers slice it (inference/kernel.py:525-526, 550).  The device twin is allocated on first use.
rms = torch.zeros((500,), dtype=torch.int64, device="cpu")
rms_gpu = None


def RMS_Norm_int64(A: torch.Tensor, W: torch.Tensor, eps, dim, host_rms=True):
    """C = floor(A * W / rms) per row, rms = isqrt((eps + sum a^2) // dim).  Returns (C, rms buffer): the 500-row host
    buffer of the reference (inference/kernel.py:525, 550).  host_rms=False (not in the reference) returns the 500-row
    DEVICE buffer instead and does not wait for the GPU: a caller that only dumps the statistic (saveTensor takes device
    tensors) keeps the layer asynchronous."""
    global rms, rms_gpu
    assert A.dtype == torch.int64
    assert A.is_cuda and W.is_cuda
    assert A.ndim == 2
    M, N = A.shape
    assert M <= rms.shape[0], "the rms buffer holds 500 rows, as in the reference"
    if rms_gpu is None or rms_gpu.device != A.device:
        rms_gpu = torch.zeros((500,), dtype=torch.int64, device=A.device)
    C = torch.empty((M, N), dtype=torch.int64, device=A.device)
    if W.dtype == torch.int32:
        lib.rms_norm_fused_32(A.data_ptr(), W.data_ptr(), rms_gpu.data_ptr(), C.data_ptr(), M, N, eps, dim)
    else:
        assert W.dtype == torch.int64
        lib.rms_norm_fused_64(A.data_ptr(), W.data_ptr(), rms_gpu.data_ptr(), C.data_ptr(), M, N, eps, dim)
    _check("RMS_Norm_int64")
    if not host_rms:
        return (C, rms_gpu)
    rms[:M] = rms_gpu[:M].cpu()
    return (C, rms)


def RMS_Norm_residual_int64(X: torch.Tensor, Y: torch.Tensor, k: int, W: torch.Tensor, eps, dim, inplace=False, host_rms=True):
    """The residual connection and the norm behind it in one pass over the row (inference/model.py:1465-1468,
    1472 with the next block's :1453): X' = X + Y * 2^k in wrapping int64, C = RMSNorm(X') with weights W.
    Returns (X', C, rms buffer); inplace=True writes X' over X."""
    global rms, rms_gpu
    assert X.dtype == torch.int64 and Y.dtype == torch.int64 and X.shape == Y.shape
    assert X.is_cuda and Y.is_cuda and W.is_cuda and X.is_contiguous() and Y.is_contiguous()
    assert X.ndim == 2
    M, N = X.shape
    assert M <= rms.shape[0], "the rms buffer holds 500 rows, as in the reference"
    if rms_gpu is None or rms_gpu.device != X.device:
        rms_gpu = torch.zeros((500,), dtype=torch.int64, device=X.device)
    Xout = X if inplace else torch.empty_like(X)
    C = torch.empty((M, N), dtype=torch.int64, device=X.device)
    assert W.dtype in (torch.int32, torch.int64)
    fn = lib.rms_norm_residual_fused_32 if W.dtype == torch.int32 else lib.rms_norm_residual_fused_64
    fn(X.data_ptr(), Y.data_ptr(), k, W.data_ptr(), Xout.data_ptr(), rms_gpu.data_ptr(), C.data_ptr(), M, N, eps, dim)
    _check("RMS_Norm_residual_int64")
    if not host_rms:
        return (Xout, C, rms_gpu)
    rms[:M] = rms_gpu[:M].cpu()
    return (Xout, C, rms)


def quantize_fp8_weight(weight: torch.Tensor, scale: torch.Tensor, k: int) -> torch.Tensor:
    """int32 fixed-point weights from a block-scaled fp8 checkpoint tensor, in one pass on the device:
    (weight_dequant(weight, scale).to(float32) * 2**k).round().to(int32) of inference/convert2.py:144-147
    (weight_dequant: inference/kernel.py:96-117, 128x128 blocks, bfloat16 result).
    weight [rows, cols] float8_e4m3fn (or its bytes as uint8), scale [ceil(rows/128), ceil(cols/128)] float32."""
    assert weight.is_cuda and scale.is_cuda and weight.is_contiguous() and scale.is_contiguous()
    assert weight.dim() == 2 and scale.dim() == 2
    assert weight.dtype in (torch.float8_e4m3fn, torch.uint8) and scale.dtype == torch.float32
    rows, cols = weight.shape
    assert scale.shape == ((rows + 127) // 128, (cols + 127) // 128)
    out = torch.empty((rows, cols), dtype=torch.int32, device=weight.device)
    lib.fp8_block_scaled_to_int32(weight.data_ptr(), scale.data_ptr(), out.data_ptr(), rows, cols, k)
    _check("quantize_fp8_weight")
    return out


def quantize_bf16(param: torch.Tensor, k: int, dtype=torch.int32) -> torch.Tensor:
    """(param.to(float32) * 2**k).round().to(dtype) for a bfloat16 tensor (inference/convert2.py:250-262, 290-295,
    353-359), dtype int32 or int64."""
    assert param.is_cuda and param.is_contiguous() and param.dtype == torch.bfloat16
    assert dtype in (torch.int32, torch.int64)
    out = torch.empty(param.shape, dtype=dtype, device=param.device)
    fn = lib.bf16_scaled_round_to_int32 if dtype == torch.int32 else lib.bf16_scaled_round_to_int64
    fn(param.data_ptr(), out.data_ptr(), param.numel(), k)
    _check("quantize_bf16")
    return out


atexit.register(lambda: lib.zk_dump_flush())


LOG_TABLE_SIZE = 8
EXP2_FRAC_LUT_Q21 = None
EXP2_FRAC_LUT_Q19 = None
EXP2_FRAC_LUT_Q25 = None
EXP2_FRAC_LUT_Q23 = None


def _host_table(init_fn):
    table = torch.zeros((2 ** LOG_TABLE_SIZE,), dtype=torch.int64, device="cpu")
    init_fn(table.data_ptr())
    return table


def softmax_init_q21():
    global EXP2_FRAC_LUT_Q21
    EXP2_FRAC_LUT_Q21 = _host_table(lib.softmax_init_q21).cuda()


def softmax_init_q19():
    global EXP2_FRAC_LUT_Q19
    EXP2_FRAC_LUT_Q19 = _host_table(lib.softmax_init_q19).cuda()


def silu_init_q25():
    global EXP2_FRAC_LUT_Q25
    EXP2_FRAC_LUT_Q25 = _host_table(lib.silu_init_q25).cuda()


def silu_init_q23():
    global EXP2_FRAC_LUT_Q23
    EXP2_FRAC_LUT_Q23 = _host_table(lib.silu_init_q23).cuda()


def _softmax(fn, name, R, C, lut):
    assert R.is_cuda and C.is_cuda
    assert lut is not None, "call the matching *_init_* first"
    Bsz, S, H, T = R.shape
    fn(R.data_ptr(), C.data_ptr(), lut.data_ptr(), Bsz, S, H, T)
    _check(name)


def softmax_q21(R: torch.Tensor, C: torch.Tensor):
    _softmax(lib.softmax_q21, "softmax_q21", R, C, EXP2_FRAC_LUT_Q21)


def softmax_q19(R: torch.Tensor, C: torch.Tensor):
    _softmax(lib.softmax_q19, "softmax_q19", R, C, EXP2_FRAC_LUT_Q19)


def _act(fn, name, R, C, lut):
    assert R.is_cuda and C.is_cuda
    assert lut is not None, "call the matching *_init_* first"
    Bsz, S, Dim = R.shape
    fn(R.data_ptr(), C.data_ptr(), lut.data_ptr(), Bsz, S, Dim)
    _check(name)


def silu_q25(R: torch.Tensor, C: torch.Tensor):
    _act(lib.silu_q25, "silu_q25", R, C, EXP2_FRAC_LUT_Q25)


def sigmoid_q25(R: torch.Tensor, C: torch.Tensor):
    _act(lib.sigmoid_q25, "sigmoid_q25", R, C, EXP2_FRAC_LUT_Q25)


def silu_q23(R: torch.Tensor, C: torch.Tensor):
    _act(lib.silu_q23, "silu_q23", R, C, EXP2_FRAC_LUT_Q23)


def sigmoid_q23(R: torch.Tensor, C: torch.Tensor):
    _act(lib.sigmoid_q23, "sigmoid_q23", R, C, EXP2_FRAC_LUT_Q23)


# ---- fusions (no counterpart in the reference's kernel.py: each replaces a kernel call plus the tensor ops around it)
def softmax_q19_scores(s1, s2, mask, C, scores=None, mul=94, div=695):
    """C = softmax_q19(floor((s1 + s2) * mul / div) + mask[None, :, None, :]) in one pass over [Bsz,S,H,T]; the
    prepared scores are also written to `scores` when given (inference/model.py:896-915).  s2 and mask may be None."""
    assert s1.is_cuda and C.is_cuda and s1.dtype == torch.int64 and s1.is_contiguous() and C.is_contiguous()
    assert EXP2_FRAC_LUT_Q19 is not None, "call softmax_init_q19 first"
    Bsz, S, H, T = s1.shape
    for t in (s2, scores):
        assert t is None or (t.is_cuda and t.dtype == torch.int64 and t.is_contiguous() and tuple(t.shape) == (Bsz, S, H, T))
    assert mask is None or (mask.is_cuda and mask.dtype == torch.int64 and mask.is_contiguous() and tuple(mask.shape) == (S, T))
    ptr = lambda t: 0 if t is None else t.data_ptr()
    lib.softmax_q19_scores(s1.data_ptr(), ptr(s2), ptr(mask), ptr(scores), C.data_ptr(), EXP2_FRAC_LUT_Q19.data_ptr(),
                           Bsz, S, H, T, int(mul), int(div))
    _check("softmax_q19_scores")


def saveTensor(fileName, t):
    """The reference's saveTensor (inference/model.py:94-102) without the wait: the raw C-order bytes of `t` go to
    `fileName` through the library's dump writer.  Device tensors are copied behind the work already queued on the GPU,
    so `t` may be overwritten or freed right after this returns; host tensors are copied before it returns.  Call
    `dump_flush()` before reading the files (it also runs at interpreter exit)."""
    t = t.detach()
    if not t.is_contiguous():
        t = t.contiguous()
    nbytes = t.numel() * t.element_size()
    fn = lib.zk_dump_device if t.is_cuda else lib.zk_dump_host
    if fn(os.fsencode(fileName), t.data_ptr(), nbytes) != 0:
        _check("saveTensor")
    # a temporary made contiguous above stays alive until the copy is queued: device copies are stream ordered and
    # torch's allocator only hands the memory to work queued later; host data has been copied already


def dump_flush():
    """wait until every tensor passed to saveTensor is in its file; raises if any write failed"""
    if lib.zk_dump_flush() != 0:
        _check("dump_flush")


def gate_route(scores, bias, n_groups, topk_groups, topk, raw_weights=None):
    """Routing of Gate.forward on the device (inference/model.py:1143-1208): scores [T,E] int64 from sigmoid_q23, bias
    [E] int32 or None -> (weights [T,topk] int64, indices [T,topk] int64).  `raw_weights`, if given, receives the
    winners' unbiased scores (what the reference dumps as gate_weights.bin)."""
    assert scores.is_cuda and scores.dtype == torch.int64 and scores.is_contiguous() and scores.dim() == 2
    assert bias is None or (bias.is_cuda and bias.dtype == torch.int32 and bias.is_contiguous() and bias.numel() == scores.shape[1])
    T, E = scores.shape
    weights = torch.empty((T, topk), dtype=torch.int64, device=scores.device)
    indices = torch.empty((T, topk), dtype=torch.int64, device=scores.device)
    lib.gate_route_q23(scores.data_ptr(), 0 if bias is None else bias.data_ptr(), weights.data_ptr(), indices.data_ptr(),
                       0 if raw_weights is None else raw_weights.data_ptr(), T, E, n_groups, topk_groups, topk)
    _check("gate_route_q23")
    return weights, indices


def gate_sigmoid_route(logits, bias, n_groups, topk_groups, topk, raw_weights=None, keep_scores=True):
    """sigmoid_q23 and the routing of Gate.forward in one launch (inference/model.py:1135-1208): logits [T,E] int64 (the
    gate's linear output, Q23) -> (scores [T,E] or None, weights [T,topk], indices [T,topk]).  `scores` is what the
    reference keeps as original_scores and dumps as sigmoid_gate_y.bin; keep_scores=False skips writing it."""
    assert logits.is_cuda and logits.dtype == torch.int64 and logits.is_contiguous() and logits.dim() == 2
    assert bias is None or (bias.is_cuda and bias.dtype == torch.int32 and bias.is_contiguous() and bias.numel() == logits.shape[1])
    assert EXP2_FRAC_LUT_Q23 is not None, "call silu_init_q23 first"
    T, E = logits.shape
    scores = torch.empty_like(logits) if keep_scores else None
    weights = torch.empty((T, topk), dtype=torch.int64, device=logits.device)
    indices = torch.empty((T, topk), dtype=torch.int64, device=logits.device)
    lib.gate_sigmoid_route_q23(logits.data_ptr(), EXP2_FRAC_LUT_Q23.data_ptr(), 0 if bias is None else bias.data_ptr(),
                               0 if scores is None else scores.data_ptr(), weights.data_ptr(), indices.data_ptr(),
                               0 if raw_weights is None else raw_weights.data_ptr(), T, E, n_groups, topk_groups, topk)
    _check("gate_sigmoid_route_q23")
    return scores, weights, indices


# ---- MoE dispatch on the device (replaces the Python loop over the experts of MoE.forward, model.py:1325-1383)
def pointer_table(tensors):
    """device array with the addresses of the experts' weight matrices (keep the tensors alive while it is used)"""
    return torch.tensor([t.data_ptr() for t in tensors], dtype=torch.int64, device="cuda")


def moe_dispatch(indices, n_experts):
    """indices [T,K] int64 -> dict of int32 device tensors: seg [E+1], token [T*K], pos [T,K], tiles, ntiles"""
    assert indices.is_cuda and indices.dtype == torch.int64 and indices.is_contiguous() and indices.dim() == 2
    T, K = indices.shape
    i32 = lambda n: torch.empty((n,), dtype=torch.int32, device=indices.device)
    d = {"seg": i32(n_experts + 1), "token": i32(T * K), "pos": i32(T * K), "tiles": i32(2 * (T * K // 32 + n_experts)),
         "ntiles": i32(1), "rows": T * K, "groups": n_experts}
    counts = i32(n_experts)
    lib.moe_dispatch(indices.data_ptr(), T, K, n_experts, counts.data_ptr(), d["seg"].data_ptr(), d["token"].data_ptr(),
                     d["pos"].data_ptr(), d["tiles"].data_ptr(), d["ntiles"].data_ptr())
    _check("moe_dispatch")
    d["pos"] = d["pos"].view(T, K)
    return d


def moe_gather_rows(x, disp):
    """x [T,N] int64 -> [T*K,N]: the rows of x in the sorted (by expert) order of `disp`"""
    assert x.is_cuda and x.dtype == torch.int64 and x.is_contiguous() and x.dim() == 2
    out = torch.empty((disp["rows"], x.shape[1]), dtype=torch.int64, device=x.device)
    lib.moe_gather_rows(x.data_ptr(), disp["token"].data_ptr(), out.data_ptr(), disp["rows"], x.shape[1])
    _check("moe_gather_rows")
    return out


def int64_grouped_bmm(A, b_table, b32, N, c_rescale, disp, want_remainder=False):
    """A [rows,K] int64 sorted by expert, b_table = pointer_table(weights [N,K]) -> C [rows,N] (and R): every expert's
    segment of rows times that expert's matrix, with the semantics of int64_bmm_broadcast per segment"""
    assert A.is_cuda and A.dtype == torch.int64 and A.is_contiguous() and A.shape[0] == disp["rows"]
    assert b_table.is_cuda and b_table.dtype == torch.int64 and b_table.numel() == disp["groups"]
    rows, Kd = A.shape
    C = torch.empty((rows, N), dtype=torch.int64, device=A.device)
    R = torch.empty((rows, N), dtype=torch.int64, device=A.device) if want_remainder else None
    lib.int64_grouped_bmm_launcher(A.data_ptr(), b_table.data_ptr(), 1 if b32 else 0, C.data_ptr(), 0 if R is None else R.data_ptr(),
                                   c_rescale, disp["seg"].data_ptr(), disp["tiles"].data_ptr(), disp["ntiles"].data_ptr(),
                                   disp["groups"], rows, Kd, N)
    _check("int64_grouped_bmm")
    return (C, R) if want_remainder else C


def moe_combine(ye, weights, disp, T, shift=23):
    """ye [T*K,N] expert outputs in sorted order, weights [T,K] -> y [T,N] = sum_k (ye[pos[t,k]] * weights[t,k]) >> shift"""
    assert ye.is_cuda and weights.is_cuda and ye.is_contiguous() and weights.is_contiguous() and weights.dtype == torch.int64
    K = weights.shape[1]
    y = torch.empty((T, ye.shape[1]), dtype=torch.int64, device=ye.device)
    lib.moe_combine(ye.data_ptr(), weights.data_ptr(), disp["pos"].data_ptr(), y.data_ptr(), T, K, ye.shape[1], shift)
    _check("moe_combine")
    return y


def moe_experts(x, weights, indices, w1_table, w3_table, w2_table, b32, inter, c13, c2, dump_dir=None):
    """The routed-expert part of MoE.forward (inference/model.py:1355-1381) without the Python loop: x [T,dim] Q23
    activations, (weights, indices) from the gate, pointer tables of the experts' w1/w3 [inter,dim] and w2 [dim,inter]
    -> y [T,dim] = sum over each token's experts of (w2 . ((silu(w1 . x) * (w3 . x)) >> 23) * weight) >> 23.
    dump_dir: the layer's witness directory.  The reference's Expert_int writes `expert_{i}_silu_x.bin` (w1 . x of the
    expert's tokens, in token order) and `expert_{i}_silu_y.bin` (its SiLU) for every expert that has tokens
    (inference/model.py:1269-1274); here they are the experts' segments of the sorted intermediates, handed to the dump
    writer without a copy.  The segment table is read back for that (one wait, in dump mode only)."""
    T, dim = x.shape
    E = w1_table.numel()
    disp = moe_dispatch(indices.contiguous(), E)
    xs = moe_gather_rows(x.contiguous(), disp)
    g = int64_grouped_bmm(xs, w1_table, b32, inter, c13, disp)
    u = int64_grouped_bmm(xs, w3_table, b32, inter, c13, disp)
    h = torch.empty_like(g)
    s = torch.empty_like(g) if dump_dir is not None else None
    silu_mul_q23(g.unsqueeze(0), u.unsqueeze(0), h.unsqueeze(0), S=None if s is None else s.unsqueeze(0))
    if dump_dir is not None:
        seg = disp["seg"].cpu().tolist()
        for i in range(E):
            if seg[i + 1] > seg[i]:
                saveTensor(os.path.join(dump_dir, "expert_%d_silu_x.bin" % i), g[seg[i]:seg[i + 1]])
                saveTensor(os.path.join(dump_dir, "expert_%d_silu_y.bin" % i), s[seg[i]:seg[i + 1]])
    ye = int64_grouped_bmm(h, w2_table, b32, dim, c2, disp)
    return moe_combine(ye, weights.contiguous(), disp, T)


def silu_mul_q23(R, U, C, S=None):
    """C = (silu_q23(R) * U) >> 23 in one pass; the SiLU values go to S when given (inference/model.py:1039-1048)."""
    assert R.is_cuda and U.is_cuda and C.is_cuda and R.shape == U.shape == C.shape
    assert R.is_contiguous() and U.is_contiguous() and C.is_contiguous() and (S is None or S.is_contiguous())
    assert EXP2_FRAC_LUT_Q23 is not None, "call silu_init_q23 first"
    Bsz, Sq, Dim = R.shape
    lib.silu_mul_q23(R.data_ptr(), U.data_ptr(), 0 if S is None else S.data_ptr(), C.data_ptr(),
                     EXP2_FRAC_LUT_Q23.data_ptr(), Bsz, Sq, Dim)
    _check("silu_mul_q23")
