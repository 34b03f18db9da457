"""Symbol producer: pooled attention scores -> the packed symbols run() and the GEMMs take.

The reference shows the procedure as a script (benchmark/test_attn_score.py:93-160: torch sort,
cumsum and searchsorted, then Triton kernels that clear the selected entries of uint8 maps, which
benchmark/test_flashomni_attention.py:254-257 transposes and packs).  Here one HIP launch goes
from the scores to the packed bits.
"""
from typing import Optional, Tuple, Union

import torch

from . import _lib
from .utils import _require_gpu_tensor


def _threshold_vector(value, count: int, device, name: str) -> torch.Tensor:
    if isinstance(value, torch.Tensor):
        t = value.to(device=device, dtype=torch.float32).reshape(-1).contiguous()
        if t.numel() != count:
            raise ValueError("%s must have %d entries, got %d" % (name, count, t.numel()))
        return t
    return torch.full((count,), float(value), dtype=torch.float32, device=device)


def sparse_symbols_from_scores(
        pooled_score: torch.Tensor, num_text_q_blocks: int,
        q_threshold: Union[float, torch.Tensor], kv_threshold: Union[float, torch.Tensor],
        num_text_kv_blocks: Optional[int] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Turn block-pooled attention scores into packed sparse symbols.

    pooled_score: ``[B, H, NQ, NK]`` float32 / bfloat16 / float16 on the GPU (the ``pooled_score``
        of benchmark/test_attn_score.py:97).
    num_text_q_blocks / num_text_kv_blocks: ``T2T`` / ``T2T_kv`` of the reference script (the
        latter defaults to the former).
    q_threshold: cumulative-probability budget of cached q blocks, a float or ``[B]`` tensor
        (``cdfthreshd`` at :101); kv_threshold: budget of skipped key blocks per row, a float or
        ``[H]`` tensor (:124).

    Returns ``(sparse_info, sparse_info_indptr, sparse_kv_info, sparse_kv_info_indptr)``: uint8
    little-endian bit-packed symbols in the layout :meth:`BatchFlashOmniFAWithRaggedKVWrapper.run`,
    :func:`flashomni_gemm` and :func:`flashomni_gemm_reduction` read, with int32 byte indptrs of
    ``B + 1`` entries.  Nothing synchronises.
    """
    _require_gpu_tensor(pooled_score, "pooled_score")
    if pooled_score.dim() != 4:
        raise ValueError("pooled_score must be [B, H, NQ, NK]")
    scores = pooled_score.contiguous()
    B, H, NQ, NK = scores.shape
    t2t = int(num_text_q_blocks)
    t2t_kv = t2t if num_text_kv_blocks is None else int(num_text_kv_blocks)
    dev = scores.device
    q_thr = _threshold_vector(q_threshold, B, dev, "q_threshold")
    kv_thr = _threshold_vector(kv_threshold, H, dev, "kv_threshold")
    info_bytes = (NQ * H + 7) // 8
    kv_bytes = (NQ * H * NK + 7) // 8
    sparse_info = torch.empty(B * info_bytes, dtype=torch.uint8, device=dev)
    sparse_kv_info = torch.empty(B * kv_bytes, dtype=torch.uint8, device=dev)
    info_indptr = torch.empty(B + 1, dtype=torch.int32, device=dev)
    kv_indptr = torch.empty(B + 1, dtype=torch.int32, device=dev)
    with _lib.device_guard(dev):
        _lib.check(_lib.lib().fo_symbols_from_scores(
            _lib.ptr(scores), _lib.dtype_code(scores.dtype), B, H, NQ, NK, t2t, t2t_kv,
            _lib.ptr(q_thr), _lib.ptr(kv_thr), _lib.ptr(sparse_info), _lib.ptr(info_indptr),
            _lib.ptr(sparse_kv_info), _lib.ptr(kv_indptr), _lib.current_stream(dev)))
    return sparse_info, info_indptr, sparse_kv_info, kv_indptr
