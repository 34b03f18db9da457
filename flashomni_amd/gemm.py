"""GEMM-Q (``flashomni_gemm``) and GEMM-O with reduction (``flashomni_gemm_reduction``).

Signatures and defaults are those of the reference (flashomni/gemm.py:156-216); the work runs in
hand-written MFMA kernels behind the C ABI (fo_gemm_q / fo_gemm_o)."""
import torch

from . import _lib
from .utils import _require_gpu_tensor


def _check_gemm_operands(A: torch.Tensor, B: torch.Tensor, name: str):
    _require_gpu_tensor(A, "A")
    _require_gpu_tensor(B, "B")
    if A.dim() != 3 or B.dim() != 2:
        # reference: csrc/gemm.cu:26-31
        raise RuntimeError(f"{name}: A must be [B, M, K] and B must be [N, K]")
    if A.shape[2] != B.shape[1]:
        raise RuntimeError(f"{name}: K mismatch, A is {tuple(A.shape)} and B is {tuple(B.shape)}")
    if A.dtype != B.dtype or A.dtype not in (torch.bfloat16, torch.float16):
        raise RuntimeError(f"{name}: A and B must both be bfloat16 or float16")
    if not (A.is_contiguous() and B.is_contiguous()):
        raise RuntimeError(f"{name}: A and B must be contiguous")


def _symbols(sparse_info, sparse_info_indptr, device, name, batch, m, num_qo_heads,
             num_text_tokens, sparse_q_size):
    """Packed symbols and their byte offsets on ``device``.  The kernels read bit
    ``((num_text_tokens + row) // sparse_q_size) * num_qo_heads + head`` of a request's segment, so
    a segment shorter than the last such bit is refused here (the offsets themselves live on the
    device and are not read back)."""
    if sparse_info is None:
        return None, None
    if sparse_info_indptr is None:
        raise RuntimeError(f"{name}: sparse_info needs sparse_info_indptr")
    info, indptr = sparse_info, sparse_info_indptr
    if info.device != device or info.dtype != torch.uint8 or not info.is_contiguous():
        info = info.to(device=device, dtype=torch.uint8).contiguous()
    if indptr.device != device or indptr.dtype != torch.int32 or not indptr.is_contiguous():
        indptr = indptr.to(device=device, dtype=torch.int32).contiguous()
    if indptr.numel() != batch + 1:
        raise RuntimeError(f"{name}: sparse_info_indptr must have batch + 1 = {batch + 1} entries, "
                           f"got {indptr.numel()}")
    if m > 0:
        last_block = (num_text_tokens + m - 1) // sparse_q_size
        need = ((last_block + 1) * num_qo_heads + 7) // 8
        if info.numel() < need:
            raise RuntimeError(f"{name}: sparse_info holds {info.numel()} bytes, a request needs {need} "
                               f"({last_block + 1} token blocks x {num_qo_heads} heads)")
    return info, indptr


# Scratch of the GEMMs (GEMM-Q's tile list, GEMM-O's work-item cursors).  Eager calls share one
# buffer per (device, stream): calls on one stream run in order, calls on different streams may
# overlap and get their own.  A call made while its stream is being captured into a graph gets a
# buffer of its own from the allocator (the graph's memory pool then owns it for as long as the
# graph lives), and a buffer that has become too small is kept, not freed, when a larger one
# replaces it: a launch already recorded or in flight may still hold its address.  Sizes are
# rounded up to powers of two, so a stream retires at most a few dozen small buffers.
_workspaces = {}


def _gemm_workspace(device, stream, nbytes):
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
    bufs = _workspaces.setdefault((device.index, stream), [])
    if not bufs or bufs[-1].numel() < nbytes:
        bufs.append(torch.empty(1 << (max(nbytes, 4096) - 1).bit_length(), dtype=torch.uint8, device=device))
    return bufs[-1]


def flashomni_gemm(
    A: torch.Tensor,
    B: torch.Tensor,
    num_qo_heads: int,
    sparse_info: torch.Tensor = None,
    sparse_info_indptr: torch.Tensor = None,
    num_text_tokens: int = 512,
    bias: torch.Tensor = None,
    out: torch.Tensor = None,
    sparse_q_size: int = 128,
    is_full: bool = False,
    *,
    quant_out=None,
) -> torch.Tensor:
    """``out[b, tile] = A[b] @ B.T + bias`` for every (128-token block, 128-column) tile whose
    ``sparse_info`` bit is 1; the other tiles of ``out`` are left untouched (a fresh ``out`` is
    ``torch.empty``, as in the reference).

    ``quant_out`` (keyword-only extension, heads of width 128): ``(q8, scale)``, ``(q8, scale, q8_lo)``,
    ``True`` or ``"residual"`` (allocate two resp. three outputs).  The
    computed tiles are also written as fp8 e4m3fn with one absmax scale per (head, 128-token block),
    taken from the fp32 results before they are rounded: ``q8`` ``[B, M, N]`` float8_e4m3fn and
    ``scale`` ``[H, B * ceil(M / 128)]`` float32, the operands
    :meth:`BatchFlashOmniFAWithRaggedKVWrapper.run` takes as ``q`` and ``q_scale`` (what
    :func:`quant_fp8_block` would make of ``out`` in a second pass); ``q8_lo`` is the rounding
    residual of ``q8`` under the same scale (``q_lo`` of ``run``).  With ``quant_out`` given and
    ``out=False`` the 16-bit result is not written at all.  Returns ``out``, or ``(out, q8, scale)``
    resp. ``(out, q8, scale, q8_lo)`` when ``quant_out`` is given (``out`` is None if it was not
    written)."""
    _check_gemm_operands(A, B, "flashomni_gemm")
    skip_out = out is False
    if skip_out:
        if quant_out is None:
            raise RuntimeError("flashomni_gemm: out=False needs quant_out")
        out = None
    elif out is None:
        out = torch.empty((A.shape[0], A.shape[1], B.shape[0]), device=A.device, dtype=A.dtype)
    elif out.shape != (A.shape[0], A.shape[1], B.shape[0]) or out.dtype != A.dtype \
            or not out.is_contiguous() or out.device != A.device:
        raise RuntimeError("flashomni_gemm: out must be a contiguous [B, M, N] tensor of A's dtype")
    if bias is not None:
        if bias.dtype != A.dtype or bias.numel() != B.shape[0] or bias.device != A.device:
            raise RuntimeError("flashomni_gemm: bias must be [N] with A's dtype on A's device")
        bias = bias.contiguous()
    if num_qo_heads <= 0 or B.shape[0] % num_qo_heads != 0 or num_text_tokens < 0 or sparse_q_size <= 0:
        raise RuntimeError("flashomni_gemm: N must be a multiple of num_qo_heads; num_text_tokens >= 0; "
                           "sparse_q_size > 0")
    info, indptr = (None, None) if is_full else _symbols(
        sparse_info, sparse_info_indptr, A.device, "flashomni_gemm", A.shape[0], A.shape[1],
        num_qo_heads, num_text_tokens, sparse_q_size)
    if not is_full and info is None:
        raise RuntimeError("flashomni_gemm: sparse_info is required unless is_full=True")
    L = _lib.lib()
    ws_bytes = L.fo_gemm_workspace_bytes(A.shape[0], A.shape[1], B.shape[0])
    stream = _lib.current_stream(A.device)
    workspace = _gemm_workspace(A.device, stream, ws_bytes)
    if quant_out is None:
        with _lib.device_guard(A.device):
            _lib.check(L.fo_gemm_q(
                _lib.ptr(A), _lib.ptr(B), _lib.ptr(bias), _lib.ptr(out), _lib.dtype_code(A.dtype),
                A.shape[0], A.shape[1], B.shape[0], A.shape[2], sparse_q_size, num_qo_heads,
                _lib.ptr(info), _lib.ptr(indptr), num_text_tokens, int(bool(is_full)),
                _lib.ptr(workspace), ws_bytes, stream))
        return out
    Bsz, M, N = A.shape[0], A.shape[1], B.shape[0]
    n_blk = Bsz * ((M + 127) // 128)
    q8_lo = None
    if quant_out is True or quant_out == "residual":
        q8 = torch.empty((Bsz, M, N), dtype=torch.float8_e4m3fn, device=A.device)
        scale = torch.empty((num_qo_heads, n_blk), dtype=torch.float32, device=A.device)
        if quant_out == "residual":
            q8_lo = torch.empty_like(q8)
    else:
        if len(quant_out) == 3:
            q8, scale, q8_lo = quant_out
            if q8_lo.shape != (Bsz, M, N) or q8_lo.dtype not in (torch.float8_e4m3fn, torch.uint8) \
                    or not q8_lo.is_contiguous() or q8_lo.device != A.device:
                raise RuntimeError("flashomni_gemm: quant_out[2] must be a contiguous [B, M, N] float8_e4m3fn "
                                   "tensor")
        else:
            q8, scale = quant_out
        if q8.shape != (Bsz, M, N) or q8.dtype not in (torch.float8_e4m3fn, torch.uint8) \
                or not q8.is_contiguous() or q8.device != A.device:
            raise RuntimeError("flashomni_gemm: quant_out[0] must be a contiguous [B, M, N] float8_e4m3fn tensor")
        if scale.shape != (num_qo_heads, n_blk) or scale.dtype != torch.float32 \
                or not scale.is_contiguous() or scale.device != A.device:
            raise RuntimeError("flashomni_gemm: quant_out[1] must be a contiguous [H, B * ceil(M / 128)] "
                               "float32 tensor")
    with _lib.device_guard(A.device):
        _lib.check(L.fo_gemm_q_quant(
            _lib.ptr(A), _lib.ptr(B), _lib.ptr(bias), _lib.ptr(out), _lib.ptr(q8), _lib.ptr(q8_lo),
            _lib.ptr(scale), _lib.dtype_code(A.dtype), Bsz, M, N, A.shape[2], sparse_q_size, num_qo_heads,
            _lib.ptr(info), _lib.ptr(indptr), num_text_tokens, int(bool(is_full)),
            _lib.ptr(workspace), ws_bytes, stream))
    return (out, q8, scale) if q8_lo is None else (out, q8, scale, q8_lo)


def flashomni_gemm_reduction(
    A: torch.Tensor,
    B: torch.Tensor,
    num_qo_heads: int,
    sparse_info: torch.Tensor,
    sparse_info_indptr: torch.Tensor,
    num_text_tokens: int,
    bias: torch.Tensor = None,
    is_for_cache: bool = False,
    sparse_q_size: int = 128,
    out_dtype: torch.dtype = None,
) -> torch.Tensor:
    """GEMM-O.  ``is_for_cache=True``: returns ``bias[N] + sum over cached heads (bit 0)`` of
    ``A[:, :, head slice] @ B[:, head slice].T``.  ``is_for_cache=False``: ``bias`` is the cached
    ``[B, M, N]`` partial and the heads with bit 1 are added to it.

    ``out_dtype`` (extension; the reference always returns ``A.dtype``): pass ``torch.float32``
    to keep the cached partial in fp32; the second call accepts an fp32 ``bias`` matrix."""
    _check_gemm_operands(A, B, "flashomni_gemm_reduction")
    if sparse_info is None or sparse_info_indptr is None:
        raise RuntimeError("flashomni_gemm_reduction: sparse_info and sparse_info_indptr are required")
    out_dtype = A.dtype if out_dtype is None else out_dtype
    if out_dtype not in (A.dtype, torch.float32):
        raise RuntimeError("flashomni_gemm_reduction: out_dtype must be A.dtype or float32")
    Bsz, M, _ = A.shape
    N = B.shape[0]
    out = torch.empty((Bsz, M, N), device=A.device, dtype=out_dtype)
    kind = _lib.FO_BIAS_NONE
    bias_code = _lib.dtype_code(A.dtype)
    if bias is not None:
        if bias.device != A.device:
            raise RuntimeError("flashomni_gemm_reduction: bias must be on A's device")
        if is_for_cache:
            if bias.numel() != N or bias.dtype != A.dtype:
                raise RuntimeError("flashomni_gemm_reduction: with is_for_cache=True bias must be [N] "
                                   "with A's dtype")
            kind = _lib.FO_BIAS_VECTOR
        else:
            if bias.numel() != Bsz * M * N or bias.dtype not in (A.dtype, torch.float32):
                raise RuntimeError("flashomni_gemm_reduction: with is_for_cache=False bias must be "
                                   "the cached [B, M, N] partial (A's dtype or float32)")
            kind = _lib.FO_BIAS_MATRIX
            bias_code = _lib.dtype_code(bias.dtype)
        bias = bias.contiguous()
    if num_qo_heads <= 0 or num_text_tokens < 0 or sparse_q_size <= 0:
        raise RuntimeError("flashomni_gemm_reduction: num_qo_heads > 0, num_text_tokens >= 0 and "
                           "sparse_q_size > 0 are required")
    info, indptr = _symbols(sparse_info, sparse_info_indptr, A.device, "flashomni_gemm_reduction",
                            Bsz, M, num_qo_heads, num_text_tokens, sparse_q_size)
    L = _lib.lib()
    # (the reduction visits every token block and needs no tile list; long launches keep their
    # work-item cursors in the first bytes of the stream's scratch buffer)
    stream = _lib.current_stream(A.device)
    ws_bytes = 256
    workspace = _gemm_workspace(A.device, stream, ws_bytes)
    with _lib.device_guard(A.device):
        _lib.check(L.fo_gemm_o(
            _lib.ptr(A), _lib.ptr(B), _lib.ptr(bias), _lib.ptr(out), _lib.dtype_code(A.dtype), kind,
            bias_code, _lib.dtype_code(out_dtype), Bsz, M, N, A.shape[2], sparse_q_size, num_qo_heads,
            _lib.ptr(info), _lib.ptr(indptr), num_text_tokens, int(bool(is_for_cache)),
            _lib.ptr(workspace), ws_bytes, stream))
    return out
