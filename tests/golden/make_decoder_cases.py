"""Writes tests/golden/decoder_cases.json: small symbol-decoder cases with their expected work
lists.  Expected values come from a plain per-bit loop over the packed bytes (bit = 1 keep,
little-endian, flag bit qb*H+h, keep bit (qb*H+h)*NKV+kvb, per-request byte offsets) -- the
conventions of the reference kernel, include/flashomni/attention/prefill.cuh:1284-1294,1380-1403.
Run from the repository root:  python tests/golden/make_decoder_cases.py"""
import json
import os
import random


def pack_little(bits):
    out = [0] * ((len(bits) + 7) // 8)
    for i, b in enumerate(bits):
        out[i // 8] |= (1 if b else 0) << (i % 8)
    return out


def make_case(name, heads, qo_lens, kv_lens, p_active, p_keep, seed, block_q=128, block_kv=128):
    rnd = random.Random(seed)
    info_bytes, keep_bytes, info_indptr, keep_indptr = [], [], [0], [0]
    rows, ptr, idx = [], [0], []
    for r, (ql, kl) in enumerate(zip(qo_lens, kv_lens)):
        nq, nk = -(-ql // block_q), -(-kl // block_kv)
        info = [rnd.random() < p_active for _ in range(nq * heads)]
        keep = [rnd.random() < p_keep for _ in range(nq * heads * nk)]
        for qb in range(nq):
            for h in range(heads):
                if info[qb * heads + h]:
                    rows.append([r, qb, h])
                    idx += [kb for kb in range(nk) if keep[(qb * heads + h) * nk + kb]]
                    ptr.append(len(idx))
        info_bytes += pack_little(info)
        keep_bytes += pack_little(keep)
        info_indptr.append(len(info_bytes))
        keep_indptr.append(len(keep_bytes))
    qo_indptr, kv_indptr = [0], [0]
    for ql, kl in zip(qo_lens, kv_lens):
        qo_indptr.append(qo_indptr[-1] + ql)
        kv_indptr.append(kv_indptr[-1] + kl)
    return dict(name=name, heads=heads, block_q=block_q, block_kv=block_kv, qo_indptr=qo_indptr,
                kv_indptr=kv_indptr, sparse_info=info_bytes or [0], sparse_kv_info=keep_bytes or [0],
                info_indptr=info_indptr, kv_info_indptr=keep_indptr,
                expected=dict(rows=rows, kv_row_ptr=ptr, kv_idx=idx))


CASES = [
    make_case("h2_nq3_nkv5_single", 2, [300], [600], 0.7, 0.5, 1),
    make_case("ragged_two_requests", 2, [300, 130], [600, 200], 0.7, 0.5, 2),
    make_case("all_rows_active_no_kv", 3, [256], [384], 1.1, -1.0, 3),
    make_case("all_ones", 2, [256, 128], [1024 + 5, 128], 1.1, 1.1, 4),
    make_case("all_cached", 2, [384], [384], -1.0, 0.5, 5),
    make_case("nkv_13_rows_cross_bytes", 5, [640], [13 * 128 - 3], 0.6, 0.4, 6),
    make_case("tiny_lengths", 1, [1, 1, 129], [1, 257, 127], 0.8, 0.6, 7),
    make_case("nkv_67_long_rows", 3, [129], [128 * 67 + 5], 0.9, 0.1, 8),
]

if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "decoder_cases.json")
    with open(path, "w") as f:
        json.dump(CASES, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")
