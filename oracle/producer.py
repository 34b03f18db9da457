"""Symbol producer: pooled attention scores -> sparse_info / sparse_kv_info.

Test infrastructure only (see oracle/__init__.py).

Restates, in numpy fp32, the procedure the reference shows in
benchmark/test_attn_score.py:93-160 (torch sort / cumsum / searchsorted followed by the Triton
fill kernels of :5-91):

  * q symbols (:96-106): the text rows' scores towards the image key blocks are summed over
    heads and text q blocks, soft-maxed over the image key blocks, sorted ascending; the blocks
    whose cumulative mass stays <= the request's threshold are cached (symbol 0) for every head.
    The fill kernel stores at ``T2T + index`` (:58-65).
  * kv symbols (:117-128): each image q row's scores are soft-maxed over all key blocks, sorted
    ascending; the key blocks whose cumulative mass stays <= the head's threshold are skipped
    (symbol 0).  Text q rows keep every key block (:75-83, :160).

Ties between equal scores are broken by the lower index (a stable sort); torch.sort leaves that
order open, so equal scores are "parity unpinned" against the reference.  The cumulative sums are
sequential fp32 sums in sorted order (torch.cumsum's association on a GPU is not specified
either): a row whose cumulative mass comes within rounding of the threshold may select one
element more or fewer in another implementation.  `selection_bounds` gives the fp64 interval of
admissible counts that tests use for such rows.
"""
import numpy as np


def softmax_f32(x):
    """torch.softmax(-1) in fp32."""
    x = np.asarray(x, dtype=np.float32)
    e = np.exp(x - x.max(axis=-1, keepdims=True), dtype=np.float32)
    return (e / e.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float32)


def ascending_order(scores):
    """Indices of a stable ascending sort of the last axis (test_attn_score.py:98, :121)."""
    return np.argsort(np.asarray(scores), axis=-1, kind="stable")


def num_to_select(probs, order, threshold):
    """searchsorted(cumsum(sorted probs), threshold, right=True) -- test_attn_score.py:99-105.

    probs, order: [..., n]; threshold broadcastable to probs.shape[:-1].  Returns int64 counts."""
    sorted_p = np.take_along_axis(np.asarray(probs, dtype=np.float32), order, axis=-1)
    cdf = np.cumsum(sorted_p, axis=-1, dtype=np.float32)
    thr = np.broadcast_to(np.asarray(threshold, dtype=np.float32), cdf.shape[:-1])
    return (cdf <= thr[..., None]).sum(axis=-1).astype(np.int64)


def selection_bounds(scores, threshold, eps=1e-5):
    """Admissible counts [lo, hi] for every row, from an fp64 softmax and cumulative sum:
    lo = #{cdf <= thr - eps}, hi = #{cdf <= thr + eps}."""
    x = np.asarray(scores, dtype=np.float64)
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    p = e / e.sum(axis=-1, keepdims=True)
    cdf = np.cumsum(np.sort(p, axis=-1), axis=-1)
    thr = np.broadcast_to(np.asarray(threshold, dtype=np.float64), cdf.shape[:-1])[..., None]
    return (cdf <= thr - eps).sum(axis=-1), (cdf <= thr + eps).sum(axis=-1)


def fill_sparse_info(sparse_info, num_sel, sorted_indices, t2t=0):
    """triton_fill_sparse_info_kernel, test_attn_score.py:53-73: for every head,
    sparse_info[b, h, t2t + sorted_indices[b, i]] = 0 for i < num_sel[b]."""
    out = np.array(sparse_info, copy=True)
    for b in range(out.shape[0]):
        idx = np.asarray(sorted_indices[b][: int(num_sel[b])], dtype=np.int64)
        out[b][:, t2t + idx] = 0
    return out


def fill_sparse_kv_info(sparse_kv_info, num_sel, sorted_indices, t2t=0):
    """triton_fill_sparse_kv_info_kernel, test_attn_score.py:75-91: num_sel and sorted_indices
    cover the q rows from t2t on; row q of them clears entries of row q + t2t."""
    out = np.array(sparse_kv_info, copy=True)
    batch, heads, n_rows = np.asarray(num_sel).shape
    for b in range(batch):
        for h in range(heads):
            for q in range(n_rows):
                idx = np.asarray(sorted_indices[b, h, q][: int(num_sel[b, h, q])], dtype=np.int64)
                out[b, h, q + t2t, idx] = 0
    return out


def fill_flashomni(sparse_kv_info, num_kv_sel, sorted_kv_indices, sparse_info, num_q_sel,
                   sorted_q_indices, t2t=0):
    """triton_fill_flashomni_kernel, test_attn_score.py:5-51: both maps in one launch; here
    num_kv_sel / sorted_kv_indices cover every q row and rows below t2t are left alone."""
    kv = np.array(sparse_kv_info, copy=True)
    batch, heads, n_q, _ = kv.shape
    for b in range(batch):
        for h in range(heads):
            for q in range(t2t, n_q):
                idx = np.asarray(sorted_kv_indices[b, h, q][: int(num_kv_sel[b, h, q])],
                                 dtype=np.int64)
                kv[b, h, q, idx] = 0
    return kv, fill_sparse_info(sparse_info, num_q_sel, sorted_q_indices, t2t)


def q_symbols(pooled_score, t2t, t2t_kv, q_threshold):
    """test_attn_score.py:96-106.  pooled_score [B, H, NQ, NK] -> uint8 [B, H, NQ]."""
    s = np.asarray(pooled_score, dtype=np.float32)
    batch, heads, n_q, _ = s.shape
    t2i = s[:, :, :t2t, t2t_kv:].sum(axis=(1, 2), dtype=np.float32)
    probs = softmax_f32(t2i)
    order = ascending_order(t2i)
    n_sel = num_to_select(probs, order, np.asarray(q_threshold, dtype=np.float32).reshape(-1))
    ones = np.ones((batch, heads, n_q), dtype=np.uint8)
    return fill_sparse_info(ones, n_sel, order, t2t)


def kv_symbols(pooled_score, t2t, kv_threshold):
    """test_attn_score.py:117-128.  pooled_score [B, H, NQ, NK] -> uint8 [B, H, NQ, NK]."""
    s = np.asarray(pooled_score, dtype=np.float32)
    batch, heads, n_q, n_k = s.shape
    rows = s[:, :, t2t:, :]
    probs = softmax_f32(rows)
    order = ascending_order(rows)
    thr = np.asarray(kv_threshold, dtype=np.float32).reshape(1, heads, 1)
    n_sel = num_to_select(probs, order, np.broadcast_to(thr, rows.shape[:-1]))
    ones = np.ones((batch, heads, n_q, n_k), dtype=np.uint8)
    return fill_sparse_kv_info(ones, n_sel, order, t2t)


def to_kernel_layout(sparse_info, sparse_kv_info):
    """[B, H, NQ] / [B, H, NQ, NK] maps -> the flat per-request order the kernels read
    (q block major, then head: benchmark/utils.py:83-84), as uint8 [B, NQ*H] / [B, NQ*H*NK]."""
    si = np.asarray(sparse_info)
    kv = np.asarray(sparse_kv_info)
    batch = si.shape[0]
    return (np.ascontiguousarray(si.transpose(0, 2, 1)).reshape(batch, -1),
            np.ascontiguousarray(kv.transpose(0, 2, 1, 3)).reshape(batch, -1))
