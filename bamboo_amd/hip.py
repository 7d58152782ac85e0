"""ctypes binding of ``libbamboo_hip.so`` (the C ABI declared in ``include/bamboo_hip.h``).

The library is the only compute path of this package: if it is missing, loading raises,
and every wrapper raises :class:`HipKernelError` when the library reports a failure.
Tensors are passed as raw device pointers (``tensor.data_ptr()``); torch is used only to
own device memory and streams.
"""
import ctypes
import os
from ctypes import POINTER, Structure, byref, c_char_p, c_float, c_int, c_int32, c_int64, c_uint32, c_uint64, c_void_p

import torch

F32, BF16 = 0, 1
NT, NN, TN = 0, 1, 2
EPI_NONE, EPI_ACT, EPI_DACT, EPI_RESIDUAL, EPI_MUL, EPI_ACT_DACT, EPI_MUL_POS = 0, 1, 2, 3, 4, 5, 6
ACT_RELU, ACT_GELU_TANH = 0, 1
MASK_NONE, MASK_CAUSAL, MASK_KEY_PADDING = 0, 1, 2
LN_STANDARD, LN_ANNOTATED = 0, 1

ACT_CODES = {"relu": ACT_RELU, "gelu_tanh": ACT_GELU_TANH}
MASK_CODES = {"none": MASK_NONE, "causal": MASK_CAUSAL, "key_padding": MASK_KEY_PADDING}
LN_CODES = {"standard": LN_STANDARD, "annotated": LN_ANNOTATED}

EXPORTS = (
    "bb_version", "bb_last_error", "bb_init", "bb_gemm", "bb_gemm_grouped", "bb_gemm_splitk_workspace", "bb_gemm_grouped_splitk", "bb_gemm_variant", "bb_layernorm_fwd",
    "bb_layernorm_bwd_workspace", "bb_layernorm_bwd", "bb_layernorm_bwd_static", "bb_colsum_workspace", "bb_colsum_acc", "bb_rowsum_fwd", "bb_rowsum_bwd", "bb_dropout_apply", "bb_dropout_keep_host",
    "bb_softmax_fwd", "bb_softmax_bwd", "bb_attention_fwd", "bb_attention_bwd", "bb_residual_add", "bb_sqrt_one_minus_fwd", "bb_sqrt_one_minus_bwd", "bb_act_fwd", "bb_bn_workspace", "bb_batchnorm_fwd", "bb_batchnorm_bwd", "bb_patch3x3", "bb_patch3x3_strided", "bb_subsample", "bb_conv3x3_supported", "bb_conv3x3", "bb_gemm_strip_stats_supported", "bb_strip_stats_workspace", "bb_batchnorm_fwd_strips", "bb_bn_bwd_strips_workspace", "bb_gemm_bn_bwd_supported", "bb_gemm_bn_bwd", "bb_conv3x3_dgrad_bn", "bb_batchnorm_bwd_strips", "bb_batchnorm_bwd_strip_sums", "bb_mse_workspace", "bb_mse_fwd_bwd", "bb_graph_begin", "bb_graph_end", "bb_graph_launch", "bb_graph_destroy",
    "bb_adam_multi", "bb_adam_multi_scaled", "bb_grad_clip_workspace", "bb_grad_clip_coef", "bb_cast", "bb_fill_f32",
)


class HipKernelError(RuntimeError):
    pass


class GemmDesc(Structure):
    _fields_ = [
        ("layout", c_int32), ("dtype", c_int32), ("c_dtype", c_int32),
        ("M", c_int32), ("N", c_int32), ("K", c_int32),
        ("A", c_void_p), ("lda", c_int64),
        ("B", c_void_p), ("ldb", c_int64),
        ("C", c_void_p), ("ldc", c_int64),
        ("nb1", c_int32), ("nb2", c_int32),
        ("sA1", c_int64), ("sA2", c_int64), ("sB1", c_int64), ("sB2", c_int64),
        ("sC1", c_int64), ("sC2", c_int64),
        ("alpha", c_float), ("epilogue", c_int32), ("act", c_int32), ("accumulate", c_int32),
        ("bias", c_void_p), ("aux_in", c_void_p), ("aux_out", c_void_p), ("resid", c_void_p),
        ("ldaux", c_int64), ("colsum_out", c_void_p), ("colsum_ws", c_void_p),
        ("conv_h", c_int32), ("conv_w", c_int32), ("conv_c", c_int32), ("conv_row0", c_int32),
        ("strip_stats", c_void_p),
        ("dropout_p", c_float), ("dropout_k0", c_uint32), ("dropout_k1", c_uint32),
    ]


class BnBwdStats(Structure):
    _fields_ = [("x", c_void_p), ("mean", c_void_p), ("rstd", c_void_p), ("strips", c_void_p)]


def library_path():
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libbamboo_hip.so")


_lib = None


def lib():
    """Load (once) and return the shared library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise HipKernelError(
            f"{path} is missing: build it with `make -C bamboo_amd/csrc` (or __graft_entry__.build()); "
            "there is no fallback compute path")
    L = ctypes.CDLL(path)
    L.bb_last_error.restype = c_char_p
    L.bb_version.restype = c_int
    L.bb_init.restype = c_int
    L.bb_gemm.argtypes = [POINTER(GemmDesc), c_void_p]
    L.bb_gemm_grouped.argtypes = [POINTER(GemmDesc), c_int, c_void_p]
    L.bb_gemm_splitk_workspace.argtypes = [POINTER(GemmDesc), c_int]
    L.bb_gemm_splitk_workspace.restype = c_int64
    L.bb_gemm_grouped_splitk.argtypes = [POINTER(GemmDesc), c_int, c_void_p, c_int64, c_void_p]
    L.bb_gemm_variant.argtypes = [POINTER(GemmDesc), c_char_p, c_int]
    L.bb_layernorm_fwd.argtypes = [c_int, c_int, c_int, c_int, c_float, c_void_p, c_void_p, c_void_p,
                                   c_void_p, c_void_p, c_void_p, c_void_p]
    L.bb_layernorm_bwd_workspace.argtypes = [c_int]
    L.bb_layernorm_bwd_workspace.restype = c_int64
    L.bb_layernorm_bwd.argtypes = [c_int, c_int, c_int, c_int, c_float] + [c_void_p] * 11
    L.bb_layernorm_bwd_static.argtypes = [c_int, c_int, c_int, c_int, c_float] + [c_void_p] * 10
    L.bb_rowsum_fwd.argtypes = [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]
    L.bb_rowsum_bwd.argtypes = [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]
    L.bb_colsum_workspace.argtypes = [c_int]
    L.bb_colsum_workspace.restype = c_int64
    L.bb_colsum_acc.argtypes = [c_int, c_int, c_int, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]
    L.bb_softmax_fwd.argtypes = [c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]
    L.bb_softmax_bwd.argtypes = [c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]
    L.bb_attention_fwd.argtypes = [c_int] * 6 + [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_void_p,
                                   c_void_p, c_float, c_uint32, c_uint32, c_void_p]
    L.bb_attention_bwd.argtypes = [c_int] * 6 + [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64,
                                   c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_float, c_uint32,
                                   c_uint32, c_void_p]
    L.bb_dropout_apply.argtypes = [c_int, c_int64, c_void_p, c_void_p, c_float, c_uint32, c_uint32, c_void_p]
    L.bb_dropout_keep_host.argtypes = [c_float, c_uint32, c_uint32, c_uint64]
    L.bb_residual_add.argtypes = [c_int, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]
    L.bb_sqrt_one_minus_fwd.argtypes = [c_int, c_int64, c_void_p, c_void_p, c_void_p]
    L.bb_sqrt_one_minus_bwd.argtypes = [c_int, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_void_p]
    L.bb_graph_begin.argtypes = [c_void_p]
    L.bb_graph_end.argtypes = [c_void_p, POINTER(c_void_p)]
    L.bb_graph_launch.argtypes = [c_void_p, c_void_p]
    L.bb_graph_destroy.argtypes = [c_void_p]
    L.bb_act_fwd.argtypes = [c_int, c_int, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]
    L.bb_bn_workspace.argtypes = [c_int]
    L.bb_bn_workspace.restype = c_int64
    L.bb_batchnorm_fwd.argtypes = [c_int, c_int, c_int, c_float, c_float, c_int] + [c_void_p] * 11
    L.bb_batchnorm_bwd.argtypes = [c_int, c_int, c_int] + [c_void_p] * 12
    L.bb_patch3x3.argtypes = [c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]
    L.bb_patch3x3_strided.argtypes = [c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]
    L.bb_subsample.argtypes = [c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]
    L.bb_conv3x3_supported.argtypes = [c_int] * 7
    L.bb_conv3x3.argtypes = [c_int] * 7 + [c_void_p] * 5
    L.bb_gemm_strip_stats_supported.argtypes = [POINTER(GemmDesc)]
    L.bb_strip_stats_workspace.argtypes = [c_int, c_int]
    L.bb_strip_stats_workspace.restype = c_int64
    L.bb_batchnorm_fwd_strips.argtypes = [c_int, c_int, c_int, c_float, c_float, c_int] + [c_void_p] * 11
    L.bb_bn_bwd_strips_workspace.argtypes = [c_int, c_int]
    L.bb_bn_bwd_strips_workspace.restype = c_int64
    L.bb_gemm_bn_bwd_supported.argtypes = [POINTER(GemmDesc)]
    L.bb_gemm_bn_bwd.argtypes = [POINTER(GemmDesc), POINTER(BnBwdStats), c_void_p]
    L.bb_conv3x3_dgrad_bn.argtypes = [c_int] * 6 + [c_void_p] * 4 + [POINTER(BnBwdStats), c_void_p]
    L.bb_batchnorm_bwd_strips.argtypes = [c_int, c_int, c_int] + [c_void_p] * 10
    L.bb_batchnorm_bwd_strip_sums.argtypes = [c_int, c_int, c_int] + [c_void_p] * 8
    L.bb_mse_workspace.restype = c_int64
    L.bb_mse_fwd_bwd.argtypes = [c_int, c_int64, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int,
                                 c_void_p, c_void_p]
    L.bb_adam_multi.argtypes = [c_int, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int64), c_float, c_float,
                                c_float, c_float, c_int, c_int, c_int, c_float, c_int, c_void_p]
    L.bb_adam_multi_scaled.argtypes = L.bb_adam_multi.argtypes[:-1] + [c_void_p, c_void_p]
    L.bb_grad_clip_workspace.argtypes = [c_int, POINTER(c_int64)]
    L.bb_grad_clip_workspace.restype = c_int64
    L.bb_grad_clip_coef.argtypes = [c_int, POINTER(c_void_p), POINTER(c_int64), c_float, c_void_p, c_void_p, c_void_p]
    L.bb_cast.argtypes = [c_int, c_int, c_int64, c_void_p, c_void_p, c_void_p]
    L.bb_fill_f32.argtypes = [c_void_p, c_int64, c_float, c_void_p]
    _lib = L
    return L


def check(rc, what):
    if rc != 0:
        raise HipKernelError(f"{what} failed ({rc}): {lib().bb_last_error().decode()}")


def init():
    """Verify the current device is a gfx950 part."""
    check(lib().bb_init(), "bb_init")


def dtype_code(dt):
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    raise HipKernelError(f"unsupported dtype {dt}: the kernels take float32 or bfloat16")


def stream_ptr(stream=None):
    if stream is None:
        stream = torch.cuda.current_stream()
    return c_void_p(stream.cuda_stream)


def _ptr(t):
    return None if t is None else c_void_p(t.data_ptr())


def _row_major(t, name):
    if t.dim() != 2 or t.stride(1) != 1:
        raise HipKernelError(f"{name}: expected a 2-D tensor with unit inner stride, got {tuple(t.shape)}/{t.stride()}")
    return t.stride(0)


# ------------------------------------------------------------------------------------- GEMM
def gemm_desc(layout, A, B, C, *, alpha=1.0, bias=None, epilogue=EPI_NONE, act=ACT_RELU, accumulate=False,
              aux_in=None, aux_out=None, resid=None, colsum_out=None, colsum_ws=None, conv=None, strip_stats=None,
              dropout=None):
    """Descriptor of C = epilogue(alpha * op(A) op(B) [+ bias]) on 2-D row-major views.
    ``conv=(h, w)`` (TN only): B is the NHWC tensor ``[pixels, c]`` whose 3x3 patch matrix ``[pixels, 9c]`` is
    the operand, gathered inside the kernel (weight gradient of a 3x3 convolution)."""
    lda, ldb, ldc = _row_major(A, "A"), _row_major(B, "B"), _row_major(C, "C")
    if conv is not None:
        if layout != TN or not B.is_contiguous():
            raise HipKernelError("gemm: conv= needs the TN layout and a contiguous NHWC tensor as B")
        K, M = A.shape; Kb, N = B.shape[0], 9 * B.shape[1]
    elif layout == NT:
        M, K = A.shape; N, Kb = B.shape
    elif layout == NN:
        M, K = A.shape; Kb, N = B.shape
    elif layout == TN:
        K, M = A.shape; Kb, N = B.shape
    else:
        raise HipKernelError(f"bad layout {layout}")
    if K != Kb or tuple(C.shape) != (M, N):
        raise HipKernelError(f"gemm shape mismatch: A{tuple(A.shape)} B{tuple(B.shape)} C{tuple(C.shape)} layout {layout}")
    if A.dtype != B.dtype:
        raise HipKernelError("gemm: A and B dtypes differ")
    d = GemmDesc()
    d.layout, d.dtype, d.c_dtype = layout, dtype_code(A.dtype), dtype_code(C.dtype)
    d.M, d.N, d.K = M, N, K
    d.A, d.lda, d.B, d.ldb, d.C, d.ldc = A.data_ptr(), lda, B.data_ptr(), ldb, C.data_ptr(), ldc
    d.nb1 = d.nb2 = 1
    if conv is not None:
        d.conv_h, d.conv_w, d.conv_c, d.conv_row0 = conv[0], conv[1], B.shape[1], 0
    d.alpha, d.epilogue, d.act, d.accumulate = alpha, epilogue, act, int(accumulate)
    ldaux = 0
    for t in (aux_in, aux_out, resid):
        if t is not None:
            if t.dtype != A.dtype or tuple(t.shape) != (M, N):
                raise HipKernelError("gemm: aux/resid tensors must be [M,N] of the operand dtype")
            ld = _row_major(t, "aux")
            if ldaux and ld != ldaux:
                raise HipKernelError("gemm: aux tensors must share one leading dimension")
            ldaux = ld
    d.ldaux = ldaux
    if bias is not None and (bias.dtype != A.dtype or bias.numel() != N):
        raise HipKernelError("gemm: bias must be [N] of the operand dtype")
    d.bias = None if bias is None else bias.data_ptr()
    d.aux_in = None if aux_in is None else aux_in.data_ptr()
    d.aux_out = None if aux_out is None else aux_out.data_ptr()
    d.resid = None if resid is None else resid.data_ptr()
    if colsum_out is not None:
        if layout != TN or colsum_out.dtype != torch.float32 or colsum_out.numel() != M:
            raise HipKernelError("gemm: colsum_out needs the TN layout and an fp32 [M] vector")
        if colsum_ws is not None and (colsum_ws.dtype != torch.float32 or colsum_ws.numel() < colsum_workspace(M)):
            raise HipKernelError("gemm: colsum_ws too small")
        d.colsum_out = colsum_out.data_ptr()
        d.colsum_ws = None if colsum_ws is None else colsum_ws.data_ptr()
    if strip_stats is not None:
        _check_strip_stats(strip_stats, M, N)
        d.strip_stats = strip_stats.data_ptr()
    if dropout is not None and dropout[0] > 0:
        # (p, (k0, k1)): dropout on the product after bias / activation, before the residual
        d.dropout_p, (d.dropout_k0, d.dropout_k1) = dropout[0], dropout[1]
    return d


def strip_stats_workspace(rows, cols):
    """fp32 elements of the per-32-row-strip column statistics a GEMM / convolution leaves for batchnorm_fwd."""
    return int(lib().bb_strip_stats_workspace(rows, cols))


def _check_strip_stats(t, rows, cols):
    if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() < strip_stats_workspace(rows, cols):
        raise HipKernelError(f"strip_stats must be a contiguous fp32 tensor of >= {strip_stats_workspace(rows, cols)} elements")


def gemm_strip_stats_supported(layout, A, B, C):
    """Whether ``gemm(layout, A, B, C, strip_stats=...)`` is taken (bf16 NT problems of the convolution shapes)."""
    return bool(lib().bb_gemm_strip_stats_supported(byref(gemm_desc(layout, A, B, C))))


def gemm(layout, A, B, C, *, stream=None, hook=None, **kw):
    """C = epilogue(alpha * op(A) op(B) [+ bias]) on 2-D row-major views (inner stride 1).
    ``hook``: optional observer called as ``hook(desc, launch, stream)`` instead of the launch; ``launch()`` performs
    the call on ``stream`` (the benchmark brackets launches with events this way).  It belongs to the caller (an
    execution context of one engine), never to the module."""
    d = gemm_desc(layout, A, B, C, **kw)
    if hook is not None:
        hook(d, lambda: check(lib().bb_gemm(byref(d), stream_ptr(stream)), "bb_gemm"), stream)
    else:
        check(lib().bb_gemm(byref(d), stream_ptr(stream)), "bb_gemm")
    return C


def gemm_splitk_workspace(descs):
    arr = (GemmDesc * len(descs))(*descs)
    return int(lib().bb_gemm_splitk_workspace(arr, len(descs)))


def gemm_grouped(descs, stream=None, splitk_ws=None, hook=None):
    """Independent GEMMs of one layout in one launch (falls back to one launch each inside the
    library when they cannot share a kernel).  With ``splitk_ws`` (a tensor of at least
    ``gemm_splitk_workspace(descs)`` bytes) problems with few output tiles and a long contraction
    are cut along the contraction and reduced in fixed order."""
    arr = (GemmDesc * len(descs))(*descs)
    if splitk_ws is not None:
        nbytes = splitk_ws.numel() * splitk_ws.element_size()
        call = lambda: check(lib().bb_gemm_grouped_splitk(arr, len(descs), _ptr(splitk_ws), nbytes, stream_ptr(stream)),
                             "bb_gemm_grouped_splitk")
    else:
        call = lambda: check(lib().bb_gemm_grouped(arr, len(descs), stream_ptr(stream)), "bb_gemm_grouped")
    if hook is not None:
        hook(descs, call, stream)
    else:
        call()


def gemm_variant(desc):
    buf = ctypes.create_string_buffer(64)
    check(lib().bb_gemm_variant(byref(desc), buf, 64), "bb_gemm_variant")
    return buf.value.decode()


def gemm_batched(layout, dtype, M, N, K, A_ptr, lda, sA, B_ptr, ldb, sB, C_ptr, ldc, sC, nb1, nb2, *,
                 c_dtype=None, alpha=1.0, stream=None):
    """Strided two-level batched GEMM on raw pointers (attention heads inside [rows, 3h] buffers).
    sA/sB/sC are (outer, inner) element strides."""
    d = GemmDesc()
    d.layout, d.dtype, d.c_dtype = layout, dtype, dtype if c_dtype is None else c_dtype
    d.M, d.N, d.K = M, N, K
    d.A, d.lda, d.B, d.ldb, d.C, d.ldc = A_ptr, lda, B_ptr, ldb, C_ptr, ldc
    d.nb1, d.nb2 = nb1, nb2
    d.sA1, d.sA2 = sA
    d.sB1, d.sB2 = sB
    d.sC1, d.sC2 = sC
    d.alpha, d.epilogue = alpha, EPI_NONE
    check(lib().bb_gemm(byref(d), stream_ptr(stream)), "bb_gemm(batched)")



# ---- operand checks: the C ABI takes raw pointers, so what a kernel and its grid assume about its operands is
# ---- verified here, before anything is launched (a tensor that is too small would be an out-of-bounds access on
# ---- the GPU)
def _like(what, ref, **tensors):
    """Every given tensor (None allowed) is contiguous and has the shape and dtype of ``ref``."""
    if not ref.is_contiguous():
        raise HipKernelError(f"{what}: operands must be contiguous, got strides {ref.stride()} for {tuple(ref.shape)}")
    for name, t in tensors.items():
        if t is None:
            continue
        if tuple(t.shape) != tuple(ref.shape) or t.dtype != ref.dtype or not t.is_contiguous():
            raise HipKernelError(f"{what}: {name} must be a contiguous {tuple(ref.shape)} tensor of {ref.dtype}, got "
                                 f"{tuple(t.shape)} {t.dtype} strides {t.stride()}")


def _vector(what, n, dtype, **tensors):
    """Every given tensor (None allowed) holds exactly ``n`` contiguous elements of ``dtype``."""
    for name, t in tensors.items():
        if t is None:
            continue
        if t.numel() != n or t.dtype != dtype or not t.is_contiguous():
            raise HipKernelError(f"{what}: {name} must hold {n} contiguous elements of {dtype}, got {tuple(t.shape)} {t.dtype}")

# ------------------------------------------------------------------------- row-wise kernels
def layernorm_fwd(x, gain, shift, y, mean, rinv, kind, eps, stream=None):
    rows, cols = x.shape
    _like("layernorm_fwd", x, y=y)
    _vector("layernorm_fwd", cols, x.dtype, gain=gain, shift=shift)
    _vector("layernorm_fwd", rows, torch.float32, mean=mean, rinv=rinv)
    check(lib().bb_layernorm_fwd(dtype_code(x.dtype), kind, rows, cols, eps, _ptr(x), _ptr(gain), _ptr(shift),
                                 _ptr(y), _ptr(mean), _ptr(rinv), stream_ptr(stream)), "bb_layernorm_fwd")


def layernorm_bwd_workspace(cols):
    return int(lib().bb_layernorm_bwd_workspace(cols))


def _check_ln_bwd(what, x, gain, mean, rinv, dy, dres, dx, dgain, dshift):
    rows, cols = x.shape
    _like(what, x, dy=dy, dres=dres, dx=dx)
    _vector(what, cols, x.dtype, gain=gain)
    _vector(what, rows, torch.float32, mean=mean, rinv=rinv)
    _vector(what, cols, torch.float32, dgain=dgain, dshift=dshift)


def layernorm_bwd(x, gain, mean, rinv, dy, dres, dx, dgain, dshift, workspace, kind, eps, stream=None):
    rows, cols = x.shape
    _check_ln_bwd("layernorm_bwd", x, gain, mean, rinv, dy, dres, dx, dgain, dshift)
    if workspace.numel() < layernorm_bwd_workspace(cols) or workspace.dtype != torch.float32:
        raise HipKernelError("layernorm_bwd: workspace too small")
    check(lib().bb_layernorm_bwd(dtype_code(x.dtype), kind, rows, cols, eps, _ptr(x), _ptr(gain), _ptr(mean),
                                 _ptr(rinv), _ptr(dy), _ptr(dres), _ptr(dx), _ptr(dgain), _ptr(dshift),
                                 _ptr(workspace), stream_ptr(stream)), "bb_layernorm_bwd")


def layernorm_bwd_static(x, gain, mean, rinv, dy, dres, dx, dgain, dshift, kind, eps, stream=None):
    """:func:`layernorm_bwd` on the library's built-in scratch array: allocates nothing, cols <= 2048, calls that
    overlap on one GPU race."""
    rows, cols = x.shape
    _check_ln_bwd("layernorm_bwd_static", x, gain, mean, rinv, dy, dres, dx, dgain, dshift)
    check(lib().bb_layernorm_bwd_static(dtype_code(x.dtype), kind, rows, cols, eps, _ptr(x), _ptr(gain), _ptr(mean),
                                        _ptr(rinv), _ptr(dy), _ptr(dres), _ptr(dx), _ptr(dgain), _ptr(dshift),
                                        stream_ptr(stream)), "bb_layernorm_bwd_static")


def rowsum_fwd(x, y, stream=None):
    """y[r] = sum of row r of x ([rows, cols] -> [rows])."""
    rows, cols = x.shape
    if y.numel() != rows or y.dtype != x.dtype:
        raise HipKernelError("rowsum_fwd: y must hold one element of x's dtype per row")
    check(lib().bb_rowsum_fwd(dtype_code(x.dtype), rows, cols, _ptr(x), _ptr(y), stream_ptr(stream)), "bb_rowsum_fwd")


def rowsum_bwd(dy, dx, stream=None):
    """dx[r, :] = dy[r]."""
    rows, cols = dx.shape
    if dy.numel() != rows or dy.dtype != dx.dtype:
        raise HipKernelError("rowsum_bwd: dy must hold one element of dx's dtype per row")
    check(lib().bb_rowsum_bwd(dtype_code(dx.dtype), rows, cols, _ptr(dy), _ptr(dx), stream_ptr(stream)), "bb_rowsum_bwd")


def colsum_workspace(cols):
    return int(lib().bb_colsum_workspace(cols))


def colsum_acc(x, out, workspace, stream=None):
    rows, cols = x.shape
    ldx = _row_major(x, "x")
    if workspace.numel() < colsum_workspace(cols) or out.dtype != torch.float32 or out.numel() != cols:
        raise HipKernelError("colsum_acc: bad workspace/out")
    check(lib().bb_colsum_acc(dtype_code(x.dtype), rows, cols, _ptr(x), ldx, _ptr(out), _ptr(workspace),
                              stream_ptr(stream)), "bb_colsum_acc")


def softmax_fwd(s, mask, key_len=None, stream=None):
    b, h, sq, sk = s.shape
    if not s.is_contiguous():
        raise HipKernelError("softmax_fwd: scores must be contiguous")
    _vector("softmax_fwd", b, torch.int32, key_len=key_len)
    check(lib().bb_softmax_fwd(dtype_code(s.dtype), mask, b, h, sq, sk, _ptr(s), _ptr(key_len),
                               stream_ptr(stream)), "bb_softmax_fwd")


def softmax_bwd(p, dp, stream=None):
    b, h, sq, sk = p.shape
    _like("softmax_bwd", p, dp=dp)
    check(lib().bb_softmax_bwd(dtype_code(p.dtype), b, h, sq, sk, _ptr(p), _ptr(dp), stream_ptr(stream)),
          "bb_softmax_bwd")


def _drop_args(dropout):
    if dropout is None or dropout[0] <= 0:
        return 0.0, 0, 0
    return float(dropout[0]), int(dropout[1][0]), int(dropout[1][1])


FUSED_HEAD_DIMS = (64, 32, 128)   # the fused attention kernels: 64- and 128-wide heads, or pairs of 32-wide heads


def _check_attention(what, qkv, batch, heads, seq, key_len, lse, out=None, d_out=None, delta=None, d_qkv=None):
    """qkv / d_qkv: [batch*seq, 3*heads*d], out / d_out: [batch*seq, heads*d] (rows may be strided views with a unit
    inner stride), lse / delta: fp32 with batch*heads*seq contiguous elements, key_len: int32 [batch]."""
    if qkv.dim() != 2 or qkv.shape[1] % (3 * heads) != 0 or qkv.shape[1] // (3 * heads) not in FUSED_HEAD_DIMS or \
            (qkv.shape[1] // (3 * heads) == 32 and heads % 2 != 0):
        raise HipKernelError(f"{what}: qkv must be [rows, 3 * heads * d] with d = 64 or 128, or d = 32 and an even number of heads; "
                             f"got {tuple(qkv.shape)} for {heads} heads")
    rows, h = batch * seq, qkv.shape[1] // 3
    for name, t, width in (("qkv", qkv, 3 * h), ("d_qkv", d_qkv, 3 * h), ("out", out, h), ("d_out", d_out, h)):
        if t is None:
            continue
        if t.dim() != 2 or tuple(t.shape) != (rows, width) or t.stride(1) != 1 or t.stride(0) < width or t.dtype != qkv.dtype:
            raise HipKernelError(f"{what}: {name} must be [{rows}, {width}] of {qkv.dtype} with unit inner stride for batch={batch} "
                                 f"heads={heads} seq={seq}, got {tuple(t.shape)} {t.dtype} strides {t.stride()}")
    _vector(what, batch * heads * seq, torch.float32, lse=lse, delta=delta)
    _vector(what, batch, torch.int32, key_len=key_len)


def attention_fwd(qkv, out, lse, batch, heads, seq, mask, key_len=None, stream=None, dropout=None):
    """qkv: [batch*seq, 3*heads*d] (Q | K | V thirds), out: [batch*seq, heads*d], lse: fp32 [batch, heads, seq]; head
    dimension d = 64 or 128, or 32 with an even number of heads.
    ``dropout=(p, (k0, k1))``: dropout on the probabilities with the decisions of that key."""
    _check_attention("attention_fwd", qkv, batch, heads, seq, key_len, lse, out=out)
    h = qkv.shape[1] // 3
    es = qkv.element_size()
    q = qkv.data_ptr()
    check(lib().bb_attention_fwd(dtype_code(qkv.dtype), mask, batch, heads, seq, qkv.shape[1] // (3 * heads),
                                 c_void_p(q), c_void_p(q + h * es), c_void_p(q + 2 * h * es), qkv.stride(0), _ptr(out),
                                 out.stride(0), _ptr(lse), _ptr(key_len), *_drop_args(dropout), stream_ptr(stream)),
          "bb_attention_fwd")


def attention_bwd(qkv, out, d_out, lse, delta, d_qkv, batch, heads, seq, mask, key_len=None, stream=None, dropout=None):
    _check_attention("attention_bwd", qkv, batch, heads, seq, key_len, lse, out=out, d_out=d_out, delta=delta, d_qkv=d_qkv)
    if d_out.stride(0) != out.stride(0):
        raise HipKernelError("attention_bwd: out and d_out must share one leading dimension")
    h = qkv.shape[1] // 3
    es = qkv.element_size()
    q, dq = qkv.data_ptr(), d_qkv.data_ptr()
    check(lib().bb_attention_bwd(dtype_code(qkv.dtype), mask, batch, heads, seq, qkv.shape[1] // (3 * heads),
                                 c_void_p(q), c_void_p(q + h * es), c_void_p(q + 2 * h * es), qkv.stride(0), _ptr(out),
                                 _ptr(d_out), out.stride(0), _ptr(lse), _ptr(delta), c_void_p(dq),
                                 c_void_p(dq + h * es), c_void_p(dq + 2 * h * es), d_qkv.stride(0), _ptr(key_len),
                                 *_drop_args(dropout), stream_ptr(stream)), "bb_attention_bwd")


def dropout_apply(src, dst, p, key, stream=None):
    """dst = src / (1 - p) where kept, 0 elsewhere; element i of the contiguous tensor is kept when
    ``dropout_keep(p, key, i)``.  The same call on a gradient is the backward."""
    if not (src.is_contiguous() and dst.is_contiguous()) or src.shape != dst.shape or src.dtype != dst.dtype:
        raise HipKernelError("dropout_apply: src and dst must be contiguous tensors of one shape and dtype")
    check(lib().bb_dropout_apply(dtype_code(src.dtype), src.numel(), _ptr(src), _ptr(dst), float(p), int(key[0]), int(key[1]),
                                 stream_ptr(stream)), "bb_dropout_apply")


def dropout_keep(p, key, index):
    """The decision for one element, evaluated on the host (no GPU needed)."""
    return bool(lib().bb_dropout_keep_host(float(p), int(key[0]), int(key[1]), int(index)))


def dropout_key(base_seed, step, micro_batch, layer_idx, site):
    """Two 32-bit key words from what identifies one dropout mask: the model's base seed, the batch counter, the
    micro-batch, the layer (global index) and the dropout site inside the layer (splitmix64 over the five)."""
    z = 0x9E3779B97F4A7C15
    for v in (base_seed, step, micro_batch, layer_idx, site):
        z = (z + (int(v) & 0xFFFFFFFFFFFFFFFF) * 0xBF58476D1CE4E5B9 + 0x9E3779B97F4A7C15) & 0xFFFFFFFFFFFFFFFF
        z ^= z >> 30
        z = (z * 0xBF58476D1CE4E5B9) & 0xFFFFFFFFFFFFFFFF
        z ^= z >> 27
        z = (z * 0x94D049BB133111EB) & 0xFFFFFFFFFFFFFFFF
        z ^= z >> 31
    return z & 0xFFFFFFFF, z >> 32


def residual_add(a, b, out, stream=None):
    _like("residual_add", a, b=b, out=out)
    check(lib().bb_residual_add(dtype_code(a.dtype), a.numel(), _ptr(a), _ptr(b), _ptr(out), stream_ptr(stream)),
          "bb_residual_add")


def sqrt_one_minus_fwd(x, m, stream=None):
    """m = sqrt(1 - x)."""
    _like("sqrt_one_minus_fwd", x, m=m)
    check(lib().bb_sqrt_one_minus_fwd(dtype_code(x.dtype), x.numel(), _ptr(x), _ptr(m), stream_ptr(stream)), "bb_sqrt_one_minus_fwd")


def sqrt_one_minus_bwd(dm, m, dx, accumulate=True, stream=None):
    """dx (+)= dm * (-1 / (2 m)) for m = sqrt(1 - x)."""
    _like("sqrt_one_minus_bwd", dm, m=m, dx=dx)
    check(lib().bb_sqrt_one_minus_bwd(dtype_code(dm.dtype), dm.numel(), _ptr(dm), _ptr(m), _ptr(dx), int(accumulate),
                                      stream_ptr(stream)), "bb_sqrt_one_minus_bwd")


def act_fwd(x, out, act, dact=None, stream=None):
    """out = act(x); dact (optional, may be x itself) receives act'(x)."""
    _like("act_fwd", x, out=out, dact=dact)
    check(lib().bb_act_fwd(dtype_code(x.dtype), act, x.numel(), _ptr(x), _ptr(out), _ptr(dact), stream_ptr(stream)),
          "bb_act_fwd")


class Graph:
    """An executable HIP graph captured from a stream (``with Graph.capture(stream) as g: ...``)."""

    def __init__(self):
        self.exec = None

    class _Capture:
        def __init__(self, graph, stream):
            self.graph, self.stream = graph, stream

        def __enter__(self):
            check(lib().bb_graph_begin(stream_ptr(self.stream)), "bb_graph_begin")
            return self.graph

        def __exit__(self, exc_type, exc, tb):
            out = c_void_p()
            rc = lib().bb_graph_end(stream_ptr(self.stream), ctypes.byref(out))
            if exc_type is None:
                check(rc, "bb_graph_end")
                self.graph.exec = out
            elif rc == 0 and out:
                lib().bb_graph_destroy(out)
            return False

    @classmethod
    def capture(cls, stream):
        return cls._Capture(cls(), stream)

    def launch(self, stream):
        check(lib().bb_graph_launch(self.exec, stream_ptr(stream)), "bb_graph_launch")

    def __del__(self):
        try:
            if self.exec:
                lib().bb_graph_destroy(self.exec)
        except Exception:
            pass


def bn_workspace(cols):
    return int(lib().bb_bn_workspace(cols))


def batchnorm_fwd(x, gamma, beta, resid, y, mean, rstd, run_mean, run_var, workspace, eps, momentum, relu, stream=None,
                  strip_stats=None):
    """``strip_stats``: the statistics the kernel that produced ``x`` left (``gemm(..., strip_stats=)``,
    ``conv3x3(..., strip_stats=)``); the statistics pass over ``x`` is then skipped."""
    rows, cols = x.shape
    _like("batchnorm_fwd", x, resid=resid, y=y)
    _vector("batchnorm_fwd", cols, x.dtype, gamma=gamma, beta=beta)
    _vector("batchnorm_fwd", cols, torch.float32, mean=mean, rstd=rstd, run_mean=run_mean, run_var=run_var)
    if strip_stats is not None:
        _check_strip_stats(strip_stats, rows, cols)
        check(lib().bb_batchnorm_fwd_strips(dtype_code(x.dtype), rows, cols, eps, momentum, int(relu), _ptr(x), _ptr(gamma),
                                            _ptr(beta), _ptr(resid), _ptr(y), _ptr(mean), _ptr(rstd), _ptr(run_mean),
                                            _ptr(run_var), _ptr(strip_stats), stream_ptr(stream)), "bb_batchnorm_fwd_strips")
        return
    if workspace.numel() < bn_workspace(cols):
        raise HipKernelError("batchnorm_fwd: workspace too small")
    check(lib().bb_batchnorm_fwd(dtype_code(x.dtype), rows, cols, eps, momentum, int(relu), _ptr(x), _ptr(gamma),
                                 _ptr(beta), _ptr(resid), _ptr(y), _ptr(mean), _ptr(rstd), _ptr(run_mean),
                                 _ptr(run_var), _ptr(workspace), stream_ptr(stream)), "bb_batchnorm_fwd")


def batchnorm_bwd(x, gamma, mean, rstd, dy, relu_out, dx, g_out, dgamma, dbeta, workspace, stream=None):
    rows, cols = x.shape
    _like("batchnorm_bwd", x, dy=dy, relu_out=relu_out, dx=dx, g_out=g_out)
    _vector("batchnorm_bwd", cols, x.dtype, gamma=gamma)
    _vector("batchnorm_bwd", cols, torch.float32, mean=mean, rstd=rstd, dgamma=dgamma, dbeta=dbeta)
    if workspace.numel() < bn_workspace(cols):
        raise HipKernelError("batchnorm_bwd: workspace too small")
    check(lib().bb_batchnorm_bwd(dtype_code(x.dtype), rows, cols, _ptr(x), _ptr(gamma), _ptr(mean), _ptr(rstd),
                                 _ptr(dy), _ptr(relu_out), _ptr(dx), _ptr(g_out), _ptr(dgamma), _ptr(dbeta),
                                 _ptr(workspace), stream_ptr(stream)), "bb_batchnorm_bwd")


def batchnorm_bwd_strip_sums(x, mean, rstd, dy, relu_out, g_out, strips, stream=None):
    """The strip sums of ``batchnorm_bwd_strips`` by a pass of their own (bf16), in the order the GEMM epilogues add them
    up: ``g_out`` (may be ``dy``) receives ``dy * (relu_out > 0)``; without a ReLU ``g`` is ``dy`` and ``g_out`` may be None."""
    rows, cols = x.shape
    _like("batchnorm_bwd_strip_sums", x, dy=dy, relu_out=relu_out, g_out=g_out)
    _vector("batchnorm_bwd_strip_sums", cols, torch.float32, mean=mean, rstd=rstd)
    if relu_out is not None and g_out is None:
        raise HipKernelError("batchnorm_bwd_strip_sums: with relu_out the masked gradient needs g_out (may be dy)")
    if strips.dtype != torch.float32 or not strips.is_contiguous() or strips.numel() < bn_bwd_strips_workspace(rows, cols):
        raise HipKernelError("batchnorm_bwd_strip_sums: strips too small")
    check(lib().bb_batchnorm_bwd_strip_sums(dtype_code(x.dtype), rows, cols, _ptr(x), _ptr(mean), _ptr(rstd), _ptr(dy),
                                            _ptr(relu_out), _ptr(g_out), _ptr(strips), stream_ptr(stream)),
          "bb_batchnorm_bwd_strip_sums")


def batchnorm_bwd_strips(x, gamma, mean, rstd, g, strips, dx, dgamma, dbeta, stream=None):
    """``batchnorm_bwd`` for a gradient ``g`` that is masked already and whose sums per strip the kernel that produced
    it left in ``strips`` (``gemm_bn_bwd`` / ``conv3x3_dgrad_bn``)."""
    rows, cols = x.shape
    _like("batchnorm_bwd_strips", x, g=g, dx=dx)
    _vector("batchnorm_bwd_strips", cols, x.dtype, gamma=gamma)
    _vector("batchnorm_bwd_strips", cols, torch.float32, mean=mean, rstd=rstd, dgamma=dgamma, dbeta=dbeta)
    if strips.dtype != torch.float32 or not strips.is_contiguous() or strips.numel() < bn_bwd_strips_workspace(rows, cols):
        raise HipKernelError("batchnorm_bwd_strips: strips too small")
    check(lib().bb_batchnorm_bwd_strips(dtype_code(x.dtype), rows, cols, _ptr(x), _ptr(gamma), _ptr(mean), _ptr(rstd),
                                        _ptr(g), _ptr(strips), _ptr(dx), _ptr(dgamma), _ptr(dbeta), stream_ptr(stream)),
          "bb_batchnorm_bwd_strips")


def _out_side(side, stride):
    return (side - 1) // stride + 1


def patch3x3(src, dst, n, h, w, c, adjoint=False, stride=1, stream=None):
    """Patch matrix of nn.Conv2d(k=3, stride, padding=1) over NHWC rows: ``dst[n*ho*wo, 9*c]`` from ``src[n*h*w, c]``;
    ``adjoint``: ``dst[n*h*w, c]`` from ``src[n*ho*wo, 9*c]``."""
    rows_in, rows_out = n * h * w, n * _out_side(h, stride) * _out_side(w, stride)
    want_src, want_dst = (rows_out * 9 * c, rows_in * c) if adjoint else (rows_in * c, rows_out * 9 * c)
    if src.numel() != want_src or dst.numel() != want_dst or not (src.is_contiguous() and dst.is_contiguous()):
        raise HipKernelError(f"patch3x3: {tuple(src.shape)} -> {tuple(dst.shape)} does not fit n={n} h={h} w={w} c={c} "
                             f"stride={stride} adjoint={adjoint}")
    check(lib().bb_patch3x3_strided(dtype_code(src.dtype), int(adjoint), n, h, w, c, stride, _ptr(src), _ptr(dst),
                                    stream_ptr(stream)), "bb_patch3x3_strided")


def subsample(src, dst, n, h, w, c, stride, adjoint=False, stream=None):
    """Rows of the pixels a strided 1x1 convolution reads: ``dst[n*ho*wo, c]`` from ``src[n*h*w, c]``; ``adjoint``:
    ``dst[n*h*w, c]`` gets ``src[n*ho*wo, c]`` ADDED at those pixels."""
    rows_in, rows_out = n * h * w, n * _out_side(h, stride) * _out_side(w, stride)
    want_src, want_dst = (rows_out * c, rows_in * c) if adjoint else (rows_in * c, rows_out * c)
    if src.numel() != want_src or dst.numel() != want_dst or src.dtype != dst.dtype or \
            not (src.is_contiguous() and dst.is_contiguous()):
        raise HipKernelError(f"subsample: {tuple(src.shape)} -> {tuple(dst.shape)} does not fit n={n} h={h} w={w} c={c} "
                             f"stride={stride} adjoint={adjoint}")
    check(lib().bb_subsample(dtype_code(src.dtype), int(adjoint), n, h, w, c, stride, _ptr(src), _ptr(dst),
                             stream_ptr(stream)), "bb_subsample")


CONV_FWD, CONV_DGRAD = 0, 1


def conv3x3_supported(dtype, mode, n, h, w, cin, cout):
    """Whether the implicit-GEMM 3x3 convolution takes this problem (else: patch matrix + GEMM)."""
    return bool(lib().bb_conv3x3_supported(dtype_code(dtype), mode, n, h, w, cin, cout))


def conv3x3(mode, src, weight, dst, n, h, w, cin, cout, strip_stats=None, stream=None, hook=None):
    """``CONV_FWD``: dst[n*h*w, cout] = conv3x3(src[n*h*w, cin]); ``CONV_DGRAD``: dst[n*h*w, cin] = the input
    gradient for src = dy[n*h*w, cout]; weight [cout, 3, 3, cin]."""
    rows = n * h * w
    want_src, want_dst = ((rows, cin), (rows, cout)) if mode == CONV_FWD else ((rows, cout), (rows, cin))
    if tuple(src.shape) != want_src or tuple(dst.shape) != want_dst or weight.numel() != 9 * cin * cout:
        raise HipKernelError(f"conv3x3: shapes {tuple(src.shape)} {tuple(weight.shape)} {tuple(dst.shape)} do not fit "
                             f"n={n} h={h} w={w} cin={cin} cout={cout} mode={mode}")
    if not (src.is_contiguous() and dst.is_contiguous() and weight.is_contiguous()):
        raise HipKernelError("conv3x3: operands must be contiguous")
    if not (src.dtype == weight.dtype == dst.dtype):
        raise HipKernelError("conv3x3: operands must share one dtype")
    if strip_stats is not None:
        _check_strip_stats(strip_stats, rows, cout)
    call = lambda: check(lib().bb_conv3x3(dtype_code(src.dtype), mode, n, h, w, cin, cout, _ptr(src), _ptr(weight),
                                          _ptr(dst), _ptr(strip_stats), stream_ptr(stream)), "bb_conv3x3")
    if hook is not None:
        hook(ConvLaunch(mode, rows, cin, cout), call, stream)
    else:
        call()


def bn_bwd_strips_workspace(rows, cols):
    """fp32 elements of the per-32-row-strip backward sums a GEMM / convolution leaves for batchnorm_bwd_strips."""
    return int(lib().bb_bn_bwd_strips_workspace(rows, cols))


def _bn_bwd_stats(what, rows, cols, dtype, x, mean, rstd, strips):
    """The checked ``bb_bn_bwd_stats`` of a [rows, cols] gradient: the kernel reads x, mean and rstd at the product's
    indices and writes one pair of sums per 32-row strip and column."""
    if tuple(x.shape) != (rows, cols) or x.dtype != dtype or not x.is_contiguous():
        raise HipKernelError(f"{what}: x must be a contiguous {(rows, cols)} tensor of {dtype}, got {tuple(x.shape)} {x.dtype}")
    _vector(what, cols, torch.float32, mean=mean, rstd=rstd)
    if strips.dtype != torch.float32 or not strips.is_contiguous() or strips.numel() < bn_bwd_strips_workspace(rows, cols):
        raise HipKernelError(f"{what}: strips must be a contiguous fp32 tensor of >= {bn_bwd_strips_workspace(rows, cols)} elements")
    return BnBwdStats(_ptr(x), _ptr(mean), _ptr(rstd), _ptr(strips))


def _bn_bwd_epilogue(relu_out, resid):
    if relu_out is not None:
        return dict(epilogue=EPI_MUL_POS, aux_in=relu_out, resid=resid)
    return dict(epilogue=EPI_RESIDUAL, resid=resid) if resid is not None else {}


def gemm_bn_bwd_supported(A, B, C, relu_out=None, resid=None):
    """Whether ``gemm_bn_bwd(A, B, C, ...)`` is taken (bf16 NN problems of the convolution shapes)."""
    return bool(lib().bb_gemm_bn_bwd_supported(byref(gemm_desc(NN, A, B, C, **_bn_bwd_epilogue(relu_out, resid)))))


def gemm_bn_bwd(A, B, C, relu_out, x, mean, rstd, strips, resid=None, stream=None, hook=None):
    """C = (A B [+ resid]) * (relu_out > 0): the input gradient of a 1x1 convolution (plus the gradient of a skip
    connection that joins it), masked by the ReLU in front of it, with the backward sums of the batch normalisation
    in front of that ReLU (input x, statistics mean / rstd) left in ``strips`` for ``batchnorm_bwd_strips``.
    ``relu_out`` None: no ReLU."""
    d = gemm_desc(NN, A, B, C, **_bn_bwd_epilogue(relu_out, resid))
    _like("gemm_bn_bwd", C, relu_out=relu_out, resid=resid)
    bn = _bn_bwd_stats("gemm_bn_bwd", C.shape[0], C.shape[1], C.dtype, x, mean, rstd, strips)
    call = lambda: check(lib().bb_gemm_bn_bwd(byref(d), byref(bn), stream_ptr(stream)), "bb_gemm_bn_bwd")
    if hook is not None:
        hook(d, call, stream)
    else:
        call()
    return C


def conv3x3_dgrad_bn(src, weight, dst, n, h, w, cin, cout, relu_out, x, mean, rstd, strips, stream=None, hook=None):
    """``conv3x3(CONV_DGRAD, ...)`` with the result masked by ``relu_out > 0`` (None: no ReLU) and the backward sums of
    the batch normalisation in front of it left in ``strips``, as ``gemm_bn_bwd``."""
    rows = n * h * w
    if tuple(src.shape) != (rows, cout) or tuple(dst.shape) != (rows, cin) or weight.numel() != 9 * cin * cout:
        raise HipKernelError(f"conv3x3_dgrad_bn: shapes {tuple(src.shape)} {tuple(weight.shape)} {tuple(dst.shape)} do not fit "
                             f"n={n} h={h} w={w} cin={cin} cout={cout}")
    if not (src.is_contiguous() and dst.is_contiguous() and weight.is_contiguous()):
        raise HipKernelError("conv3x3_dgrad_bn: operands must be contiguous")
    if not (src.dtype == weight.dtype == dst.dtype):
        raise HipKernelError("conv3x3_dgrad_bn: operands must share one dtype")
    if relu_out is not None:
        _like("conv3x3_dgrad_bn", dst, relu_out=relu_out)
    bn = _bn_bwd_stats("conv3x3_dgrad_bn", rows, cin, dst.dtype, x, mean, rstd, strips)
    call = lambda: check(lib().bb_conv3x3_dgrad_bn(dtype_code(src.dtype), n, h, w, cin, cout, _ptr(src), _ptr(weight), _ptr(dst),
                                                   _ptr(relu_out), byref(bn), stream_ptr(stream)), "bb_conv3x3_dgrad_bn")
    if hook is not None:
        hook(ConvLaunch(CONV_DGRAD, rows, cin, cout), call, stream)
    else:
        call()


class ConvLaunch:
    """What a launch observer (``hook=``) is handed for an implicit-GEMM convolution: the GEMM it amounts to."""

    def __init__(self, mode, rows, cin, cout):
        self.variant_name = "bf16_conv3x3_fwd_igemm128x64w8k64s3" if mode == CONV_FWD else "bf16_conv3x3_dgrad_igemm64x128w8k64s3"
        self.M, self.N, self.K = (rows, cout, 9 * cin) if mode == CONV_FWD else (rows, cin, 9 * cout)
        self.epilogue = EPI_NONE


def mse_workspace():
    return int(lib().bb_mse_workspace())


def mse_fwd_bwd(y, target, dy, grad_scale, loss_out, accumulate, workspace, stream=None):
    if not y.is_contiguous():
        raise HipKernelError("mse_fwd_bwd: operands must be contiguous")
    _vector("mse_fwd_bwd", y.numel(), y.dtype, target=target, dy=dy)
    if loss_out.dtype != torch.float32 or loss_out.numel() < 1 or workspace.dtype != torch.float32 or workspace.numel() < mse_workspace():
        raise HipKernelError("mse_fwd_bwd: loss_out / workspace must be fp32 (1 resp. mse_workspace() elements)")
    check(lib().bb_mse_fwd_bwd(dtype_code(y.dtype), y.numel(), _ptr(y), _ptr(target), _ptr(dy), grad_scale,
                               _ptr(loss_out), int(accumulate), _ptr(workspace), stream_ptr(stream)),
          "bb_mse_fwd_bwd")


def grad_clip_workspace(grads):
    """Floats of workspace :func:`grad_clip_coef` needs for these gradient tensors."""
    n = len(grads)
    return int(lib().bb_grad_clip_workspace(n, (c_int64 * n)(*[t.numel() for t in grads])))


def grad_clip_coef(grads, max_norm, out, workspace, stream=None):
    """out[0] = global L2 norm of the fp32 tensors ``grads``, out[1] = min(1, max_norm / (norm + 1e-6)) (both stay on the
    device: :func:`adam_multi` takes ``out[1:]`` as its ``grad_scale``)."""
    n = len(grads)
    if any(t.dtype != torch.float32 or not t.is_contiguous() for t in grads):
        raise HipKernelError("grad_clip_coef: contiguous float32 gradients expected")
    if out.dtype != torch.float32 or out.numel() < 2 or workspace.dtype != torch.float32 or \
            workspace.numel() < grad_clip_workspace(grads):
        raise HipKernelError("grad_clip_coef: out needs 2 floats, workspace grad_clip_workspace(grads) floats")
    check(lib().bb_grad_clip_coef(n, (c_void_p * n)(*[t.data_ptr() for t in grads]), (c_int64 * n)(*[t.numel() for t in grads]),
                                  float(max_norm), _ptr(out), _ptr(workspace), stream_ptr(stream)), "bb_grad_clip_coef")


def adam_multi(g, p, m, v, lowp, *, lr, beta1, beta2, eps, step, adam_w_mode=True, bias_correction=True,
               weight_decay=0.0, zero_grad=False, grad_scale=None, stream=None):
    """Lists of fp32 tensors g/p/m/v (same lengths); lowp: list of bf16 tensors or None entries, or None.
    ``grad_scale``: one-element fp32 device tensor every gradient is multiplied by before the update (clipping)."""
    n = len(p)
    arr = lambda ts: (c_void_p * n)(*[None if t is None else t.data_ptr() for t in ts])
    sizes = (c_int64 * n)(*[t.numel() for t in p])
    for a, b_, c, d in zip(g, p, m, v):
        if not (a.dtype == b_.dtype == c.dtype == d.dtype == torch.float32):
            raise HipKernelError("adam_multi: g, p, m, v must be float32")
        if not (a.numel() == b_.numel() == c.numel() == d.numel()):
            raise HipKernelError("adam_multi: size mismatch")
    lp = arr(lowp) if lowp is not None else None
    if grad_scale is not None:
        if grad_scale.dtype != torch.float32 or grad_scale.numel() < 1 or not grad_scale.is_cuda:
            raise HipKernelError("adam_multi: grad_scale must be a float32 device tensor")
        check(lib().bb_adam_multi_scaled(n, arr(g), arr(p), arr(m), arr(v), lp, sizes, lr, beta1, beta2, eps, step,
                                         1 if adam_w_mode else 0, 1 if bias_correction else 0, weight_decay,
                                         int(zero_grad), _ptr(grad_scale), stream_ptr(stream)), "bb_adam_multi_scaled")
        return
    check(lib().bb_adam_multi(n, arr(g), arr(p), arr(m), arr(v), lp, sizes, lr, beta1, beta2, eps, step,
                              1 if adam_w_mode else 0, 1 if bias_correction else 0, weight_decay,
                              int(zero_grad), stream_ptr(stream)), "bb_adam_multi")


def cast(src, dst, stream=None):
    if src.numel() != dst.numel() or not (src.is_contiguous() and dst.is_contiguous()):
        raise HipKernelError(f"cast: contiguous tensors of one size expected, got {tuple(src.shape)} -> {tuple(dst.shape)}")
    check(lib().bb_cast(dtype_code(src.dtype), dtype_code(dst.dtype), src.numel(), _ptr(src), _ptr(dst),
                        stream_ptr(stream)), "bb_cast")


def fill_f32(dst, value, stream=None):
    check(lib().bb_fill_f32(_ptr(dst), dst.numel(), value, stream_ptr(stream)), "bb_fill_f32")
