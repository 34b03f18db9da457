"""CPU: the oracle's symbol codec and decoder pinned against numpy.packbits, the reference's
docstring known-answer vectors, closed forms and the committed hand-checked decoder fixtures."""
import json
import os

import numpy as np
import pytest

import oracle

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "decoder_cases.json")


def test_packbits_docstring_known_answers():
    # flashomni/quantization.py:90-93
    assert oracle.packbits([1, 0, 1, 1, 0, 0, 1, 1]).tolist() == [0b10110011]
    # flashomni/quantization.py:133-138
    y, p = oracle.segment_packbits([1, 0, 1, 1, 0, 0, 1, 1, 1, 0, 1], [0, 4, 7, 11], "big")
    assert y.tolist() == [0b10110000, 0b100000, 0b11010000]
    assert p.tolist() == [0, 1, 2, 3]


@pytest.mark.parametrize("n", [0, 1, 7, 8, 9, 63, 64, 65, 1000])
@pytest.mark.parametrize("bitorder", ["big", "little"])
def test_packbits_equals_numpy_and_round_trips(n, bitorder):
    rng = np.random.default_rng(n)
    x = rng.random(n) < 0.5
    y = oracle.packbits(x, bitorder)
    np.testing.assert_array_equal(y, np.packbits(x.astype(np.uint8), bitorder=bitorder))
    np.testing.assert_array_equal(np.unpackbits(y, bitorder=bitorder)[:n].astype(bool), x)


def test_packbits_rejects_bad_bitorder():
    with pytest.raises(ValueError):
        oracle.packbits([1], "middle")


def test_segment_packbits_byte_alignment_and_indptr():
    rng = np.random.default_rng(1)
    lens = [0, 3, 8, 17, 0, 64]
    indptr = np.concatenate([[0], np.cumsum(lens)])
    x = rng.random(indptr[-1]) < 0.5
    y, p = oracle.segment_packbits(x, indptr, "little")
    assert (np.diff(p) == (np.array(lens) + 7) // 8).all()
    for i, n in enumerate(lens):
        seg = np.unpackbits(y[p[i]:p[i + 1]], bitorder="little")[:n].astype(bool)
        np.testing.assert_array_equal(seg, x[indptr[i]:indptr[i + 1]])


def test_indptr_helpers_closed_forms():
    # FLUX shape: 36 q-blocks x 24 heads, 36 kv blocks (bits) -> 108 / 3888 bytes
    assert oracle.sparse_info_indptr_bits([0, 4608], 24, 128).tolist() == [0, 864]
    assert oracle.sparse_kv_info_indptr_bits([0, 4608], [0, 4608], 24, 128, 128).tolist() == [0, 31104]
    assert oracle.sparse_info_indptr_bits([0, 1, 130, 130], 2, 128).tolist() == [0, 2, 6, 6]
    assert oracle.sparse_kv_info_indptr_bits([0, 1, 130], [0, 300, 301], 2, 128, 128).tolist() == [0, 6, 10]


def test_get_bit_is_little_endian():
    buf = np.array([0b00000101, 0b10000000], dtype=np.uint8)
    assert [oracle.get_bit(buf, 0, i) for i in range(16)] == [1, 0, 1, 0, 0, 0, 0, 0] + [0] * 7 + [1]
    assert oracle.get_bit(buf, 1, 7) == 1


def test_decoder_hand_written_case():
    """H=2, one request of 3 q-blocks and 5 kv blocks, worked out by hand.
    sparse_info bits (qb*H+h): 1,0, 1,1, 0,1 -> byte 0b00101101.
    keep bits, row (qb,h) = 5 bits each, bit index (qb*2+h)*5+kvb:
      (0,0) 10001  (0,1) 11111  (1,0) 00000  (1,1) 01010  (2,0) 11111  (2,1) 00100"""
    info = np.array([0b00101101], dtype=np.uint8)
    rows = ["10001", "11111", "00000", "01010", "11111", "00100"]
    bits = np.array([int(c) for r in rows for c in r], dtype=np.uint8)
    keep = np.packbits(bits, bitorder="little")
    r = oracle.decode_kv_csr(info, keep, [0, 1], [0, len(keep)], [0, 300], [0, 600], 2, 128, 128)
    assert r[0].tolist() == [0, 0, 0, 0]
    assert r[1].tolist() == [0, 1, 1, 2]          # q-blocks of the active rows
    assert r[2].tolist() == [0, 0, 1, 1]          # heads
    assert r[3].tolist() == [0, 2, 2, 4, 5]       # row (1,0) is active with no kept block
    assert r[4].tolist() == [0, 4, 1, 3, 2]


def _bruteforce(case):
    """Independent per-bit python loop (no numpy unpacking)."""
    H, bq, bk = case["heads"], case["block_q"], case["block_kv"]
    info, keep = case["sparse_info"], case["sparse_kv_info"]
    rows, ptr, idx = [], [0], []
    for r in range(len(case["qo_indptr"]) - 1):
        nq = -(-(case["qo_indptr"][r + 1] - case["qo_indptr"][r]) // bq)
        nk = -(-(case["kv_indptr"][r + 1] - case["kv_indptr"][r]) // bk)
        for qb in range(nq):
            for h in range(H):
                i = qb * H + h
                if not (info[case["info_indptr"][r] + i // 8] >> (i % 8)) & 1:
                    continue
                rows.append([r, qb, h])
                for kb in range(nk):
                    j = i * nk + kb
                    if (keep[case["kv_info_indptr"][r] + j // 8] >> (j % 8)) & 1:
                        idx.append(kb)
                ptr.append(len(idx))
    return rows, ptr, idx


def test_decoder_matches_golden_fixtures():
    cases = json.load(open(GOLDEN))
    assert len(cases) >= 5
    for case in cases:
        r = oracle.decode_kv_csr(np.array(case["sparse_info"], dtype=np.uint8),
                                 np.array(case["sparse_kv_info"], dtype=np.uint8),
                                 case["info_indptr"], case["kv_info_indptr"], case["qo_indptr"],
                                 case["kv_indptr"], case["heads"], case["block_q"], case["block_kv"])
        exp = case["expected"]
        assert np.stack(r[:3], 1).tolist() == exp["rows"], case["name"]
        assert r[3].tolist() == exp["kv_row_ptr"], case["name"]
        assert r[4].tolist() == exp["kv_idx"], case["name"]
        # the fixture itself agrees with a from-scratch per-bit loop
        rows, ptr, idx = _bruteforce(case)
        assert (rows, ptr, idx) == (exp["rows"], exp["kv_row_ptr"], exp["kv_idx"])


def test_decoder_invariants_random():
    from helpers import make_ragged_masks
    m = make_ragged_masks([300, 1, 1000], [77, 513, 4096], 3, 0.6, 0.3, seed=9)
    req, qb, head, ptr, idx = oracle.decode_kv_csr(m["packed_info"], m["packed_keep"], m["info_indptr"],
                                                   m["keep_indptr"], m["qo_indptr"], m["kv_indptr"], 3, 128, 128)
    assert len(req) == sum(int(i.sum()) for i in m["info"])
    assert ptr[-1] == sum(int((k & i[:, :, None]).sum()) for i, k in zip(m["info"], m["keep"]))
    key = req.astype(np.int64) * 10 ** 6 + qb * 1000 + head
    assert (np.diff(key) > 0).all()                       # ascending (request, q-block, head)
    for i in range(len(req)):
        seg = idx[ptr[i]:ptr[i + 1]]
        assert (np.diff(seg) > 0).all()
        np.testing.assert_array_equal(seg, np.nonzero(m["keep"][req[i]][qb[i], head[i]])[0])
    # is_full lists everything
    full = oracle.decode_kv_csr(None, None, None, None, m["qo_indptr"], m["kv_indptr"], 3, 128, 128, True)
    assert len(full[0]) == sum(i.size for i in m["info"]) and full[3][-1] == sum(k.size for k in m["keep"])


def test_head_csr_for_gemm_o():
    info = np.array([0b00101101], dtype=np.uint8)   # (qb,h): 1,0 | 1,1 | 0,1
    ptr, idx = oracle.decode_head_csr(info, [0, 1], 1, 384, 2, 128, 0, 128, want_bit=1)
    assert ptr.tolist() == [0, 1, 3, 4] and idx.tolist() == [0, 0, 1, 1]
    ptr, idx = oracle.decode_head_csr(info, [0, 1], 1, 384, 2, 128, 0, 128, want_bit=0)
    assert ptr.tolist() == [0, 1, 1, 2] and idx.tolist() == [1, 0]
    # num_text_tokens shifts the q-block (gemm_reduction.cuh:128)
    ptr, idx = oracle.decode_head_csr(info, [0, 1], 1, 256, 2, 128, 128, 128, want_bit=1)
    assert ptr.tolist() == [0, 2, 3] and idx.tolist() == [0, 1, 1]
