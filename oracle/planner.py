"""Host-side prefill planner restated in python.  Test infrastructure only.

Follows include/flashomni/attention/scheduler.cuh:35-64 (kv chunk binary search),
:67-168 (tile enumeration), :248-349 (workspace layout through the 16-byte
aligned bump allocator of include/flashomni/allocator.h:32-58) and
include/flashomni/utils.cuh:293-312 (q tile size)."""


def _ceil_div(a, b):
    return -(-a // b)


def determine_cta_tile_q(avg_packed_qo_len, head_dim):
    """utils.cuh:293-312 on an Ampere-or-newer device."""
    if avg_packed_qo_len > 64 and head_dim < 256:
        return 128
    return 64 if avg_packed_qo_len > 16 else 16


def binary_search_kv_chunk(enable_graph, max_batch_if_split, packed_qo_len, kv_len, qo_chunk,
                           min_kv_chunk):
    """scheduler.cuh:35-64."""
    high = max([1] + list(kv_len))
    max_kv_len = high
    low = min_kv_chunk
    while low < high:
        mid = (low + high) // 2
        nb = sum(_ceil_div(q, qo_chunk) * _ceil_div(max(k, 1), mid)
                 for q, k in zip(packed_qo_len, kv_len))
        if nb > max_batch_if_split:
            low = mid + 1
        else:
            high = mid
    return (enable_graph or low < max_kv_len), low


class _Bump:
    def __init__(self, size):
        self.cur, self.size = 0, size

    def alloc(self, nbytes, align):
        start = _ceil_div(self.cur, align) * align
        if start + nbytes > self.size:
            raise RuntimeError("workspace overflow")
        self.cur = start + nbytes
        return start


def prefill_plan(qo_indptr, kv_indptr, num_qo_heads, num_kv_heads, head_dim_vo, num_cu,
                 int_ws_bytes=8 * 1024 * 1024, float_ws_bytes=128 * 1024 * 1024, page_size=1, enable_graph=False, total_num_rows=None):
    """Returns dict with the 15 plan_info entries (scheduler.cuh:205-221) and the arrays."""
    if num_qo_heads % num_kv_heads:
        raise RuntimeError("num_qo_heads should be divisible by num_kv_heads")
    batch = len(qo_indptr) - 1
    group = num_qo_heads // num_kv_heads
    if total_num_rows is None:
        total_num_rows = int(qo_indptr[-1])
    packed = [int(qo_indptr[i + 1] - qo_indptr[i]) * group for i in range(batch)]
    kvl = [int(kv_indptr[i + 1] - kv_indptr[i]) for i in range(batch)]
    if min(packed + [0]) < 0 or min(kvl + [0]) < 0:
        raise RuntimeError("indptr should be non-decreasing")
    max_batch_if_split = (2 * num_cu) // num_kv_heads
    min_kv_chunk = max(128 // page_size, 1)
    if enable_graph:
        max_seq = total_num_rows - batch + 1
        cta_tile_q = determine_cta_tile_q(max_seq * group, head_dim_vo)
        total_tiles_q = _ceil_div(total_num_rows * group, cta_tile_q) + batch - 1
    else:
        cta_tile_q = determine_cta_tile_q(sum(packed) // batch, head_dim_vo)
        total_tiles_q = sum(_ceil_div(p, cta_tile_q) for p in packed)
    split_kv, kv_chunk = binary_search_kv_chunk(enable_graph, max_batch_if_split, packed, kvl,
                                                cta_tile_q, min_kv_chunk)
    req, qt, kt, o_indptr, merge = [], [], [], [0], [0]
    for r in range(batch):
        ntq = _ceil_div(packed[r], cta_tile_q)
        ntk = _ceil_div(max(kvl[r], 1), kv_chunk)
        for a in range(ntq):
            for b in range(ntk):
                req.append(r); qt.append(a); kt.append(b)
        qo_len = packed[r] // group
        for _ in range(qo_len):
            merge.append(merge[-1] + ntk)
        o_indptr.append(o_indptr[-1] + qo_len * ntk)
    new_batch = len(req)
    padded = max(max_batch_if_split, total_tiles_q) if enable_graph else new_batch
    kv_chunk *= page_size
    bump = _Bump(int_ws_bytes)
    off = {}
    off["request_indices"] = bump.alloc(4 * padded, 16)
    off["qo_tile_indices"] = bump.alloc(4 * padded, 16)
    off["kv_tile_indices"] = bump.alloc(4 * padded, 16)
    off["o_indptr"] = bump.alloc(4 * (batch + 1), 16)
    off["kv_chunk_size_ptr"] = bump.alloc(4, 1)
    off["total_num_rows"] = bump.alloc(4, 16) if enable_graph else 0
    off["merge_indptr"] = off["block_valid_mask"] = 0
    v_off = s_off = 0
    if split_kv:
        fb = _Bump(float_ws_bytes)
        v_off = fb.alloc(num_qo_heads * padded * cta_tile_q * head_dim_vo * 4, 16)
        s_off = fb.alloc(num_qo_heads * padded * cta_tile_q * 4, 16)
        off["merge_indptr"] = bump.alloc(4 * (total_num_rows + 1), 16)
        off["block_valid_mask"] = bump.alloc(padded, 16)
    info = [padded, total_num_rows, off["total_num_rows"], cta_tile_q, off["request_indices"],
            off["qo_tile_indices"], off["kv_tile_indices"], off["merge_indptr"], off["o_indptr"],
            off["kv_chunk_size_ptr"], v_off, s_off, off["block_valid_mask"], int(enable_graph), int(split_kv)]
    return dict(plan_info=info, request_indices=req, qo_tile_indices=qt, kv_tile_indices=kt,
                o_indptr=o_indptr, merge_indptr=merge, kv_chunk_size=kv_chunk, split_kv=split_kv,
                cta_tile_q=cta_tile_q, padded_batch_size=padded, used_bytes=bump.cur)
