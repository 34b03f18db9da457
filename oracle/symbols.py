"""Bit-packed sparse symbols: packing, indptr arithmetic and brute-force decode.

Test infrastructure only (see oracle/__init__.py).

Bit conventions, all taken from the reference kernels:
  * bit value 1 = compute / keep, 0 = cached / skip
    (include/flashomni/attention/prefill.cuh:1291, gemm/w16a16/gemm.cuh:55);
  * little-endian inside a byte: ``(buf[i // 8] >> (i % 8)) & 1``;
  * ``sparse_info`` bit index inside a request  = q_block * H + head
    (prefill.cuh:1285-1287);
  * ``sparse_kv_info`` bit index inside a request = (q_block * H + head) * NKV + kv_block,
    NKV = ceil(kv_len / block_kv) (prefill.cuh:1288-1290, 1385);
  * ``*_indptr`` handed to run() are BYTE offsets of each request's segment
    (flashomni/quantization.py:148-159 via benchmark/test_flashomni_attention.py:254-260).
"""
import numpy as np


def get_bit(buf, base_byte, i):
    """(buf[base + i//8] >> (i%8)) & 1 -- prefill.cuh:1291."""
    return (int(buf[base_byte + i // 8]) >> (i % 8)) & 1


def packbits(x, bitorder="big"):
    """flashomni/quantization.py:68-99, include/flashomni/quantization.cuh:39-57.

    Written out bit by bit (not numpy.packbits) so the test against
    numpy.packbits is a real cross-check."""
    if bitorder not in ("big", "little"):
        raise ValueError("bitorder must be 'big' or 'little'")
    x = np.asarray(x).astype(bool).reshape(-1)
    n = x.shape[0]
    out = np.zeros((n + 7) // 8, dtype=np.uint8)
    for j in range(8):
        part = x[j::8].astype(np.uint8)
        shift = (7 - j) if bitorder == "big" else j
        out[: part.shape[0]] |= part << shift
    return out


def segment_packbits(x, indptr, bitorder="big"):
    """flashomni/quantization.py:102-159, quantization.cuh:59-83: every segment
    starts on a byte boundary; new_indptr = cumsum((len + 7) // 8)."""
    x = np.asarray(x).astype(bool).reshape(-1)
    indptr = np.asarray(indptr).astype(np.int64)
    seglen = indptr[1:] - indptr[:-1]
    new_indptr = np.zeros_like(indptr)
    new_indptr[1:] = np.cumsum((seglen + 7) // 8)
    y = np.zeros(int(new_indptr[-1]), dtype=np.uint8)
    for i in range(len(seglen)):
        y[new_indptr[i]:new_indptr[i + 1]] = packbits(x[indptr[i]:indptr[i + 1]], bitorder)
    return y, new_indptr.astype(np.int32)


def _ceil_div(a, b):
    return -(-a // b)


def sparse_info_indptr_bits(qo_indptr, num_qo_heads, block_q):
    """flashomni/attention.py:165-176 (bit counts, not bytes)."""
    qo = np.asarray(qo_indptr).astype(np.int64)
    out = np.zeros_like(qo)
    out[1:] = np.cumsum(_ceil_div(qo[1:] - qo[:-1], block_q) * num_qo_heads)
    return out


def sparse_kv_info_indptr_bits(qo_indptr, kv_indptr, num_qo_heads, block_q, block_kv):
    """flashomni/attention.py:178-191 (bit counts, not bytes)."""
    qo = np.asarray(qo_indptr).astype(np.int64)
    kv = np.asarray(kv_indptr).astype(np.int64)
    out = np.zeros_like(qo)
    out[1:] = np.cumsum(_ceil_div(qo[1:] - qo[:-1], block_q)
                        * _ceil_div(kv[1:] - kv[:-1], block_kv) * num_qo_heads)
    return out


def _unpack_segment(buf, base_byte, nbits):
    nbytes = (nbits + 7) // 8
    seg = np.asarray(buf[base_byte:base_byte + nbytes], dtype=np.uint8)
    return np.unpackbits(seg, bitorder="little")[:nbits]


def decode_rows(sparse_info, sparse_info_indptr, qo_indptr, num_heads, block_q, is_full=False):
    """Canonical row list: every (request, q_block, head) whose sparse_info bit is 1,
    ascending in (request, q_block, head).  prefill.cuh:1284-1294.

    Returns int32 arrays (row_req, row_qb, row_head)."""
    qo = np.asarray(qo_indptr).astype(np.int64)
    req, qb, head = [], [], []
    for r in range(len(qo) - 1):
        nq = _ceil_div(int(qo[r + 1] - qo[r]), block_q)
        n = nq * num_heads
        if is_full:
            bits = np.ones(n, dtype=np.uint8)
        else:
            bits = _unpack_segment(sparse_info, int(sparse_info_indptr[r]), n)
        idx = np.nonzero(bits)[0]
        req.append(np.full(idx.shape, r))
        qb.append(idx // num_heads)
        head.append(idx % num_heads)
    cat = lambda xs: (np.concatenate(xs) if xs else np.zeros(0)).astype(np.int32)
    return cat(req), cat(qb), cat(head)


def decode_kv_csr(sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr,
                  qo_indptr, kv_indptr, num_heads, block_q, block_kv, is_full=False):
    """Canonical attention work list.  prefill.cuh:1284-1294 (row flag),
    1380-1403 and 1434-1460 (walk of the kv bits of one row).

    Returns (row_req, row_qb, row_head, kv_row_ptr[n_rows+1], kv_idx[nnz]), all int32.
    Active rows with no kept kv block stay in the list (they must write zeros,
    prefill.cuh:944-946)."""
    row_req, row_qb, row_head = decode_rows(sparse_info, sparse_info_indptr, qo_indptr,
                                            num_heads, block_q, is_full)
    kv = np.asarray(kv_indptr).astype(np.int64)
    ptr = [0]
    idx = []
    for r, qb, h in zip(row_req, row_qb, row_head):
        nkv = _ceil_div(int(kv[r + 1] - kv[r]), block_kv)
        if is_full:
            kept = np.arange(nkv)
        else:
            base = (int(qb) * num_heads + int(h)) * nkv
            first_byte = int(sparse_kv_info_indptr[r]) + base // 8
            bits = _unpack_segment(sparse_kv_info, first_byte, base % 8 + nkv)[base % 8:]
            kept = np.nonzero(bits)[0]
        idx.append(kept)
        ptr.append(ptr[-1] + len(kept))
    kv_idx = (np.concatenate(idx) if idx else np.zeros(0)).astype(np.int32)
    return row_req, row_qb, row_head, np.asarray(ptr, dtype=np.int32), kv_idx


def decode_head_csr(sparse_info, sparse_info_indptr, batch, m_rows, num_heads, block_q,
                    num_text_tokens, tile_m, want_bit):
    """GEMM-O head list per (batch, row-tile): heads whose bit == want_bit.
    gemm/w16a16/gemm_reduction.cuh:126-160 (bit index (num_text_tokens + iy*BM)/sq * H + head)."""
    ptr = [0]
    idx = []
    for b in range(batch):
        for iy in range(_ceil_div(m_rows, tile_m)):
            qb = (num_text_tokens + iy * tile_m) // block_q
            for h in range(num_heads):
                if get_bit(sparse_info, int(sparse_info_indptr[b]), qb * num_heads + h) == want_bit:
                    idx.append(h)
            ptr.append(len(idx))
    return np.asarray(ptr, dtype=np.int32), np.asarray(idx, dtype=np.int32)
