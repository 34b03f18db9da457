"""fp32 dense masked attention: the reference CPU path.  Test infrastructure only.

Semantics follow include/flashomni/attention/prefill.cuh:
  * a (request, q_block, head) whose sparse_info bit is 0 leaves `out` untouched (:1284-1294);
  * kept kv blocks are those whose sparse_kv_info bit is 1 (:1380-1403, :1434-1460);
    keys past kv_len are masked (:715-757, tail only);
  * an active row with no kept block writes zeros and lse = -5e4
    (finite "infinity" of include/flashomni/math.cuh:32; :385-386, :944-946, :1517-1520);
  * lse is base-2: log2(sum exp2(s*c - m*c)) + m*c with c = sm_scale*log2(e)
    (:973, :1517; include/flashomni/attention/variants.cuh:54);
  * logits_soft_cap > 0: the logits become tanh(q.k * sm_scale / cap) and the softmax scale
    log2(e) * cap (variants.cuh:43-56 set-up, :68-70 transform), i.e. scores cap * tanh(q.k * sm_scale / cap).
The block mask is expanded to token granularity exactly like the reference benchmark builds
its SDPA mask (benchmark/test_flashomni_attention.py:197-199): repeat_interleave(block) and crop.

Grouped-query attention (fewer kv heads than q heads, group = H / H_kv), gqa_symbols="packed_tile":
the reference's layout.  A request's q rows are its (token, q head of the group) pairs, token-major
per kv head: packed row p = token p // group, q head kv_head * group + p % group (:410-413 load,
:1128, :1178 store, :1510-1511 lse).  A launch block is (tile of 128 packed rows, kv head)
(:1273-1278); its sparse_info bit is tile * H_kv + kv_head and its kv mask starts at that bit index
times the request's number of kv blocks (:1283-1290).  gqa_symbols="per_q_head" (no reference
counterpart): symbols per (128-token block, q head), q head h reads kv head h // group.
"""
import math

import numpy as np
import torch

from .symbols import decode_kv_csr

NEG_INF = -5e4


def sparse_attention(q, k, v, sparse_info, sparse_kv_info, sparse_info_indptr,
                     sparse_kv_info_indptr, qo_indptr, kv_indptr, block_q=128, block_kv=128,
                     sm_scale=None, is_full=False, out=None, lse=None, rows=None,
                     q_scale=None, k_scale=None, q_lo=None, k_lo=None, gqa_symbols="per_q_head",
                     logits_soft_cap=0.0):
    """q [nnz_q,H,D], k/v [nnz_kv,H,D] (any float dtype; math is fp32 on the given values).

    `out` (same dtype as q unless q is fp8, then bf16) is updated in place for active rows only; allocated
    as zeros when None (flashomni/attention.py:779-785).  `rows`: optional iterable of
    row-list positions to evaluate (sampling for the big configs); others are left untouched.
    q_scale/k_scale: optional fp32 [H, n_blocks] dequantisation scales for fp8 q/k; q_lo: optional
    second fp8 term added to q before scaling; k_lo: the same for k (no reference counterpart)."""
    H, D = q.shape[1], q.shape[2]
    group = H // k.shape[1]   # q heads per kv head (prefill.cuh:410-413); 1 without grouped-query attention
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    out_dtype = q.dtype if q.dtype in (torch.float16, torch.bfloat16, torch.float32) else torch.bfloat16
    if out is None:
        out = torch.zeros(q.shape[:-1] + v.shape[-1:], dtype=out_dtype)
    to_np = lambda t: None if t is None else (t.cpu().numpy() if torch.is_tensor(t) else np.asarray(t))
    qo = to_np(qo_indptr).astype(np.int64)
    kvp = to_np(kv_indptr).astype(np.int64)
    packed = group > 1 and gqa_symbols == "packed_tile"
    if packed:
        assert q_scale is None and k_scale is None, "packed tiles take 16-bit q and k"
        return _packed_tiles(q, k, v, to_np(sparse_info), to_np(sparse_kv_info), to_np(sparse_info_indptr),
                             to_np(sparse_kv_info_indptr), qo, kvp, group, block_q, block_kv,
                             sm_scale, is_full, out, lse, rows, logits_soft_cap)
    row_req, row_qb, row_head, ptr, idx = decode_kv_csr(
        to_np(sparse_info), to_np(sparse_kv_info), to_np(sparse_info_indptr),
        to_np(sparse_kv_info_indptr), qo, kvp, H, block_q, block_kv, is_full)
    c = sm_scale * math.log2(math.e)
    # scale tensors index token blocks request by request (blocks never straddle requests)
    q_blk_base = np.concatenate([[0], np.cumsum(-(-(qo[1:] - qo[:-1]) // block_q))])
    kv_blk_base = np.concatenate([[0], np.cumsum(-(-(kvp[1:] - kvp[:-1]) // block_kv))])
    sel = range(len(row_req)) if rows is None else rows
    for i in sel:
        r, qb, h = int(row_req[i]), int(row_qb[i]), int(row_head[i])
        q0 = int(qo[r]) + qb * block_q
        q1 = min(int(qo[r + 1]), q0 + block_q)
        kv0, kv1 = int(kvp[r]), int(kvp[r + 1])
        kept = idx[ptr[i]:ptr[i + 1]]
        if len(kept) == 0:
            out[q0:q1, h] = 0
            if lse is not None:
                lse[q0:q1, h] = NEG_INF
            continue
        tok = np.concatenate([np.arange(kv0 + b * block_kv, min(kv1, kv0 + (b + 1) * block_kv))
                              for b in kept])
        tok_t = torch.from_numpy(tok)
        qf = q[q0:q1, h].float()
        if q_lo is not None:
            qf = qf + q_lo[q0:q1, h].float()
        kf = k[tok_t, h // group].float()
        if k_lo is not None:
            kf = kf + k_lo[tok_t, h // group].float()
        vf = v[tok_t, h // group].float()
        if q_scale is not None:
            qf = qf * float(q_scale[h, int(q_blk_base[r]) + qb])
        if k_scale is not None:
            blk = torch.from_numpy((tok - kv0) // block_kv + int(kv_blk_base[r]))
            kf = kf * k_scale[h // group][blk].float()[:, None]
        o_rows, lse_rows = _softmax_pv(qf @ kf.T, vf, sm_scale, logits_soft_cap)
        out[q0:q1, h] = o_rows.to(out.dtype)
        if lse is not None:
            lse[q0:q1, h] = lse_rows
    return out


def _softmax_pv(s, vf, sm_scale, logits_soft_cap):
    """Rows of raw logits s = q.k^T -> (softmax(s) @ v, base-2 lse), fp32."""
    c = sm_scale * math.log2(math.e)
    if logits_soft_cap > 0:
        # variants.cuh:47-48: soft_cap_pre_tanh_scale = sm_scale / cap, sm_scale_log2 = log2(e) * cap
        s = torch.tanh(s * (sm_scale / logits_soft_cap))
        c = math.log2(math.e) * logits_soft_cap
    m = s.max(dim=-1, keepdim=True).values
    p = torch.exp2((s - m) * c)
    d = p.sum(dim=-1, keepdim=True)
    return (p @ vf) / d, (torch.log2(d) + m * c).squeeze(-1)


def _packed_tiles(q, k, v, sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr, qo, kvp,
                  group, block_q, block_kv, sm_scale, is_full, out, lse, rows, logits_soft_cap=0.0):
    """The reference's grouped-query layout (see the module text).  The symbols of a request with
    qo_len tokens are those of an ungrouped request with qo_len * group rows and H_kv heads
    (prefill.cuh:1283-1290 with gridDim.z = H_kv), so the same decoder lists the (tile, kv head) rows."""
    H_kv = k.shape[1]
    c = sm_scale * math.log2(math.e)
    qo_packed = qo * group
    row_req, row_tile, row_kvh, ptr, idx = decode_kv_csr(
        sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr, qo_packed, kvp, H_kv,
        block_q, block_kv, is_full)
    sel = range(len(row_req)) if rows is None else rows
    for i in sel:
        r, tile, kvh = int(row_req[i]), int(row_tile[i]), int(row_kvh[i])
        qlen = int(qo[r + 1] - qo[r])
        pr = np.arange(tile * block_q, min((tile + 1) * block_q, qlen * group))   # packed rows of the tile
        tok = torch.from_numpy(int(qo[r]) + pr // group)                            # :410 divmod -> q
        hq = torch.from_numpy(kvh * group + pr % group)                             # :410 divmod -> r, :1323
        kv0, kv1 = int(kvp[r]), int(kvp[r + 1])
        kept = idx[ptr[i]:ptr[i + 1]]
        if len(kept) == 0:
            out[tok, hq] = 0
            if lse is not None:
                lse[tok, hq] = NEG_INF
            continue
        kt = torch.from_numpy(np.concatenate([np.arange(kv0 + b * block_kv, min(kv1, kv0 + (b + 1) * block_kv))
                                              for b in kept]))
        qf = q[tok, hq].float()
        kf = k[kt, kvh].float()
        vf = v[kt, kvh].float()
        o_rows, lse_rows = _softmax_pv(qf @ kf.T, vf, sm_scale, logits_soft_cap)
        out[tok, hq] = o_rows.to(out.dtype)
        if lse is not None:
            lse[tok, hq] = lse_rows
    return out
