"""packbits / segment_packbits (reference API: flashomni/quantization.py:68-159) and the fp8
block quantiser (no reference counterpart), all running as HIP kernels through the C ABI."""
from typing import Tuple

import torch

from . import _lib
from .utils import _require_gpu_tensor

_BITORDER = {"big": 0, "little": 1}


def _bitorder_code(bitorder: str) -> int:
    if bitorder not in _BITORDER:
        # same message as the reference binding (csrc/quantization.cu:25)
        raise RuntimeError("bitorder must be 'big' or 'little'")
    return _BITORDER[bitorder]


def _as_bool_bytes(x: torch.Tensor) -> torch.Tensor:
    x = x.to(torch.bool).contiguous()
    return x.view(torch.uint8)


def packbits(x: torch.Tensor, bitorder: str = "big") -> torch.Tensor:
    r"""Pack the elements of a binary-valued array into bits in a uint8 array.

    Same semantics as ``numpy.packbits``.  ``x`` is a 1D tensor on the GPU; returns a uint8
    tensor of ``(x.size(0) + 7) // 8`` bytes.

    >>> x = torch.tensor([1, 0, 1, 1, 0, 0, 1, 1], dtype=torch.bool, device="cuda")
    >>> list(map(bin, packbits(x).tolist()))
    ['0b10110011']
    """
    code = _bitorder_code(bitorder)
    _require_gpu_tensor(x, "x")
    xb = _as_bool_bytes(x.reshape(-1))
    y = torch.empty((xb.size(0) + 7) // 8, dtype=torch.uint8, device=x.device)
    with _lib.device_guard(x.device):
        _lib.check(_lib.lib().fo_packbits(_lib.ptr(xb), xb.size(0), code, _lib.ptr(y),
                                          _lib.current_stream(x.device)))
    return y


def segment_packbits(x: torch.Tensor, indptr: torch.Tensor,
                     bitorder: str = "big") -> Tuple[torch.Tensor, torch.Tensor]:
    r"""Pack a batch of binary-valued segments into bits; every segment starts on a byte.

    Returns ``(y, new_indptr)`` with
    ``new_indptr[i+1] - new_indptr[i] == (indptr[i+1] - indptr[i] + 7) // 8``.

    >>> x = torch.tensor([1, 0, 1, 1, 0, 0, 1, 1, 1, 0, 1], dtype=torch.bool, device="cuda")
    >>> y, p = segment_packbits(x, torch.tensor([0, 4, 7, 11], device="cuda"), bitorder="big")
    >>> list(map(bin, y.tolist())), p.tolist()
    (['0b10110000', '0b100000', '0b11010000'], [0, 1, 2, 3])

    The output length is data dependent, so this call synchronises with the host once
    (as the reference does, flashomni/quantization.py:152).
    """
    code = _bitorder_code(bitorder)
    _require_gpu_tensor(x, "x")
    seglen = indptr[1:] - indptr[:-1]
    packed_len = (seglen + 7) // 8
    indptr_new = torch.zeros(len(indptr), dtype=indptr.dtype, device=indptr.device)
    indptr_new[1:] = torch.cumsum(packed_len, 0)
    output_nnzs = int(indptr_new[-1].item())

    device = x.device
    indptr = indptr.to(device=device, dtype=torch.int32)
    indptr_new = indptr_new.to(device=device, dtype=torch.int32)
    xb = _as_bool_bytes(x.reshape(-1))
    y = torch.empty(output_nnzs, dtype=torch.uint8, device=device)
    with _lib.device_guard(device):
        _lib.check(_lib.lib().fo_segment_packbits(_lib.ptr(xb), _lib.ptr(indptr), _lib.ptr(indptr_new),
                                                  len(indptr) - 1, code, _lib.ptr(y),
                                                  _lib.current_stream(device)))
    return y, indptr_new


def token_blocks(indptr: torch.Tensor, block: int = 128):
    """Host helper: (first token, length) of every ``block``-token block, request by request.
    ``indptr`` is a host or device int tensor of batch+1 entries."""
    ip = indptr.to("cpu", torch.int64)
    tok0, length = [], []
    for r in range(len(ip) - 1):
        a, b = int(ip[r]), int(ip[r + 1])
        t = a
        while t < b:
            tok0.append(t)
            length.append(min(block, b - t))
            t += block
    return (torch.tensor(tok0, dtype=torch.int32), torch.tensor(length, dtype=torch.int32))


def quant_fp8_block(x: torch.Tensor, indptr: torch.Tensor, block: int = 128,
                    blocks=None, residual: bool = False):
    """Quantise ``x`` [nnz, H, D] (bf16/fp16, GPU) to fp8 e4m3fn with one absmax scale per
    (head, ``block``-token block); blocks never straddle the requests delimited by ``indptr``.

    Returns ``(x8 [nnz,H,D] float8_e4m3fn, scale [H, n_blocks] float32)`` with
    ``scale = absmax / 448`` (1 for an all-zero block) and ``x ~= x8 * scale``.
    ``blocks``: optional cached result of :func:`token_blocks` already on the GPU.
    ``residual=True`` returns ``(x8, scale, x8_lo)``: ``x8_lo`` is the rounding residual
    ``x / scale - x8`` as a second float8_e4m3fn tensor, ``x ~= (x8 + x8_lo) * scale`` to about 7
    significant bits (the ``q_lo`` operand of fp8 attention)."""
    _require_gpu_tensor(x, "x")
    if block != 128:
        raise ValueError("quant_fp8_block: only 128-token blocks are supported")
    if x.dim() != 3 or x.stride(2) != 1:
        raise ValueError("quant_fp8_block: x must be [nnz, H, D] with a contiguous last dim")
    if blocks is None:
        tok0, length = token_blocks(indptr, block)
        blocks = (tok0.to(x.device), length.to(x.device))
    tok0, length = blocks
    nnz, H, D = x.shape
    x8 = torch.empty((nnz, H, D), dtype=torch.float8_e4m3fn, device=x.device)
    x8_lo = torch.empty_like(x8) if residual else None
    scale = torch.empty((H, tok0.numel()), dtype=torch.float32, device=x.device)
    with _lib.device_guard(x.device):
        _lib.check(_lib.lib().fo_quant_fp8_block(
            _lib.ptr(x), _lib.dtype_code(x.dtype), x.stride(0), x.stride(1), _lib.ptr(x8),
            _lib.ptr(x8_lo), _lib.ptr(scale), _lib.ptr(tok0), _lib.ptr(length), tok0.numel(), H, D,
            _lib.current_stream(x.device)))
    return (x8, scale, x8_lo) if residual else (x8, scale)
