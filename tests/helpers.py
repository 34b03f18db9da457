"""Shared test helpers: random ragged problems, mask packing, error metrics."""
import numpy as np
import torch

BLOCK = 128


def ceil_div(a, b):
    return -(-a // b)


def make_ragged_masks(qo_lens, kv_lens, heads, p_active=0.75, p_keep=0.5, seed=0, force=None):
    """Random symbols for a ragged batch.  Returns dict with bool masks per request and the packed
    little-endian tensors + byte indptrs (numpy), laid out as the reference expects:
    sparse_info [q_block, head], sparse_kv_info [q_block, head, kv_block] per request."""
    rng = np.random.default_rng(seed)
    infos, keeps = [], []
    for ql, kl in zip(qo_lens, kv_lens):
        nq, nk = ceil_div(ql, BLOCK), ceil_div(kl, BLOCK)
        info = rng.random((nq, heads)) < p_active
        keep = rng.random((nq, heads, nk)) < p_keep
        if force == "ones":
            info[:] = True
            keep[:] = True
        elif force == "zeros":
            info[:] = False
        infos.append(info)
        keeps.append(keep)
    def pack(parts):
        segs = [np.packbits(p.reshape(-1).astype(np.uint8), bitorder="little") for p in parts]
        indptr = np.zeros(len(segs) + 1, dtype=np.int32)
        indptr[1:] = np.cumsum([len(s) for s in segs])
        data = np.concatenate(segs) if segs else np.zeros(0, dtype=np.uint8)
        if data.size == 0:
            data = np.zeros(1, dtype=np.uint8)
        return data, indptr
    pinfo, pinfo_indptr = pack(infos)
    pkeep, pkeep_indptr = pack(keeps)
    qo_indptr = np.zeros(len(qo_lens) + 1, dtype=np.int32)
    qo_indptr[1:] = np.cumsum(qo_lens)
    kv_indptr = np.zeros(len(kv_lens) + 1, dtype=np.int32)
    kv_indptr[1:] = np.cumsum(kv_lens)
    return dict(info=infos, keep=keeps, packed_info=pinfo, info_indptr=pinfo_indptr,
                packed_keep=pkeep, keep_indptr=pkeep_indptr, qo_indptr=qo_indptr,
                kv_indptr=kv_indptr)


def rel_l2(a, b):
    a, b = a.float(), b.float()
    return float((a - b).norm() / b.norm().clamp_min(1e-20))


def max_abs(a, b):
    return float((a.float() - b.float()).abs().max())


def sentinel_like(shape, dtype, device="cpu", seed=123):
    """A recognisable non-trivial byte pattern used to prove that skipped outputs stay untouched."""
    g = torch.Generator().manual_seed(seed)
    t = (torch.rand(shape, generator=g) * 8 - 4).to(dtype)
    return t.to(device)
