"""Masked dense GEMMs in fp32: the reference CPU path for GEMM-Q / GEMM-O.
Test infrastructure only.

GEMM-Q  include/flashomni/gemm/w16a16/gemm.cuh:50-58 (tile skip test), :83-92 (accumulator
        initialised from bias), :213-214 (single round-to-nearest cast at the end).
GEMM-O  include/flashomni/gemm/w16a16/gemm_reduction.cuh:77-95 (init = bias vector when
        caching, cached [B,M,N] matrix otherwise), :126-160 (head-slice selection).
Shape rules csrc/gemm.cu:26-36."""
import numpy as np
import torch

from .symbols import get_bit

TILE = 128


def _np(t):
    return t.cpu().numpy() if torch.is_tensor(t) else np.asarray(t)


def gemm_q(x, w, num_qo_heads, sparse_info=None, sparse_info_indptr=None, num_text_tokens=512,
           bias=None, out=None, sparse_q_size=128, is_full=False):
    """x [B,M,K], w [N,K] -> out [B,M,N]; inactive (128-row, 128-col) tiles keep `out`'s bytes."""
    B, M, K = x.shape
    N = w.shape[0]
    head_dim = N // num_qo_heads
    if out is None:
        out = torch.empty(B, M, N, dtype=x.dtype)
    wf = w.float()
    bf = None if bias is None else bias.float()
    info = None if is_full else _np(sparse_info)
    indptr = None if is_full else _np(sparse_info_indptr)
    for b in range(B):
        for iy in range(-(-M // TILE)):
            r0, r1 = iy * TILE, min(M, (iy + 1) * TILE)
            cols = []
            for ix in range(N // TILE):
                if is_full:
                    cols.append(ix)
                    continue
                bit = ((num_text_tokens + iy * TILE) // sparse_q_size) * num_qo_heads \
                    + (ix * TILE) // head_dim
                if get_bit(info, int(indptr[b]), bit):
                    cols.append(ix)
            if not cols:
                continue
            xf = x[b, r0:r1].float()
            for ix in cols:
                y = xf @ wf[ix * TILE:(ix + 1) * TILE].T
                if bf is not None:
                    y = y + bf[ix * TILE:(ix + 1) * TILE]
                out[b, r0:r1, ix * TILE:(ix + 1) * TILE] = y.to(out.dtype)
    return out


def gemm_o(x, w, num_qo_heads, sparse_info, sparse_info_indptr, num_text_tokens, bias=None,
           is_for_cache=False, sparse_q_size=128, out_dtype=None):
    """x [B,M,K] (K = H*head_dim), w [N,K] -> [B,M,N].  Every output tile is written."""
    B, M, K = x.shape
    N = w.shape[0]
    head_dim = N // num_qo_heads          # csrc/gemm_reduction.cu:32
    out = torch.empty(B, M, N, dtype=out_dtype or x.dtype)
    wf = w.float()
    info, indptr = _np(sparse_info), _np(sparse_info_indptr)
    n_slices = K // head_dim
    for b in range(B):
        for iy in range(-(-M // TILE)):
            r0, r1 = iy * TILE, min(M, (iy + 1) * TILE)
            qb = (num_text_tokens + iy * TILE) // sparse_q_size
            if bias is None:
                acc = torch.zeros(r1 - r0, N)
            elif is_for_cache:
                acc = bias.float()[None, :].expand(r1 - r0, N).clone()
            else:
                acc = bias[b, r0:r1].float().clone()
            for h in range(n_slices):
                bit = get_bit(info, int(indptr[b]), qb * num_qo_heads + h)
                if (bit == 0) == bool(is_for_cache):
                    ks = slice(h * head_dim, (h + 1) * head_dim)
                    acc += x[b, r0:r1, ks].float() @ wf[:, ks].T
            out[b, r0:r1] = acc.to(out.dtype)
    return out
