"""GPU: the decoder entry point that allocates nothing (fo_decode_sparse_static: scratch in a
built-in device array) against fo_decode_sparse on the same inputs, bit for bit, on two calls in a
row, the second on a smaller input."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import make_ragged_masks

pytestmark = pytest.mark.gpu


def _buffers(dev, max_rows, max_nnz):
    i32 = lambda n: torch.full((max(n, 1),), -7, dtype=torch.int32, device=dev)
    return dict(row_req=i32(max_rows), row_qb=i32(max_rows), row_head=i32(max_rows), kv_row_ptr=i32(max_rows + 1),
                kv_idx=i32(max_nnz), counts=i32(4), order=i32(max_rows), sched=i32(1024),
                shares=i32(512 + 8 * (max_rows + 1)))


def _decode(dev, m, heads, static, share_table):
    """Both entry points through the C ABI with identical tables; returns the outputs on the host."""
    from flashomni_amd import _lib
    L = _lib.lib()
    qo, kv = torch.from_numpy(m["qo_indptr"]), torch.from_numpy(m["kv_indptr"])
    batch = qo.numel() - 1
    sizes = torch.zeros(3, dtype=torch.int64)
    _lib.check(L.fo_decode_sizes(qo.data_ptr(), kv.data_ptr(), batch, heads, 128, 128, sizes[0:].data_ptr(),
                                 sizes[1:].data_ptr(), sizes[2:].data_ptr()))
    n_blk, max_rows, max_nnz = (int(v) for v in sizes)
    table = torch.empty((2, max(n_blk, 1)), dtype=torch.int32)
    _lib.check(L.fo_sparse_block_table(qo.data_ptr(), batch, 128, table[0].data_ptr(), table[1].data_ptr(), n_blk,
                                       sizes[0:].data_ptr()))
    table_d, kv_d = table.to(dev), kv.to(dev)
    t = lambda a: torch.from_numpy(a).to(dev)
    sym = [t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"])]
    b = _buffers(dev, max_rows, max_nnz)
    stream = torch.cuda.current_stream(dev).cuda_stream
    head = [sym[0].data_ptr(), sym[1].data_ptr(), sym[2].data_ptr(), sym[3].data_ptr(), table_d[0].data_ptr(),
            table_d[1].data_ptr(), kv_d.data_ptr(), n_blk, heads, 128, 0]
    outs = [b[n].data_ptr() for n in ("row_req", "row_qb", "row_head", "kv_row_ptr", "kv_idx", "counts", "order",
                                      "sched")]
    shares = b["shares"].data_ptr() if share_table else None
    if static:
        before = torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev)
        _lib.check(L.fo_decode_sparse_static(*head, *outs, shares, stream))
        assert (torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev)) == before
    else:
        scratch = torch.empty(2 * n_blk * heads + 8192, dtype=torch.int32, device=dev)
        _lib.check(L.fo_decode_sparse(*head, *outs, scratch.data_ptr(), shares, stream))
    torch.cuda.synchronize(dev)
    return {k: v.cpu().numpy() for k, v in b.items()}, n_blk * heads


def _assert_same(a, b):
    n_rows, nnz = int(a["counts"][0]), int(a["counts"][1])
    assert list(a["counts"]) == list(b["counts"])
    for name, n in (("row_req", n_rows), ("row_qb", n_rows), ("row_head", n_rows), ("kv_row_ptr", n_rows + 1),
                    ("kv_idx", nnz)):
        np.testing.assert_array_equal(a[name][:n], b[name][:n], err_msg=name)
    np.testing.assert_array_equal(a["sched"][:64], b["sched"][:64])
    fixed_order = a["sched"][26] != 0 or a["sched"][32] != 0
    for x in range(8):  # queue by queue (inside a length class the order is not fixed for medium lists)
        lo, hi = int(a["sched"][x]), int(a["sched"][x + 1])
        if fixed_order:
            np.testing.assert_array_equal(a["order"][lo:hi], b["order"][lo:hi])
        else:
            np.testing.assert_array_equal(np.sort(a["order"][lo:hi]), np.sort(b["order"][lo:hi]))
    if fixed_order:
        np.testing.assert_array_equal(a["shares"], b["shares"])
    return n_rows


# (q lens, kv lens, heads, p_active, p_keep): a long list (fixed ascending order), then a smaller
# one (length classes), then one small enough for even shares
CALLS = [([128 * 300 - 17, 700], [2000, 300], 12, 0.9, 0.5),
         ([4608], [4608], 24, 0.75, 0.5),
         ([1000, 129], [640, 300], 5, 0.7, 0.4)]


@pytest.mark.parametrize("share_table", [True, False])
def test_static_scratch_decoder_matches(dev, share_table):
    rows = []
    for i, (ql, kl, heads, pa, pk) in enumerate(CALLS):   # calls in a row, each smaller than the last
        m = make_ragged_masks(ql, kl, heads, pa, pk, seed=40 + i)
        got, pairs = _decode(dev, m, heads, True, share_table)
        exp, _ = _decode(dev, m, heads, False, share_table)
        rows.append((_assert_same(got, exp), pairs))
    assert rows[0][1] > rows[1][1] > rows[2][1] and rows[0][0] > rows[1][0] > rows[2][0] > 0


def test_static_scratch_decoder_refuses_large_inputs(dev):
    from flashomni_amd import _lib
    L = _lib.lib()
    limit = L.fo_decode_sparse_static_max_pairs()
    assert limit == (262144 - 8192) // 2
    one = torch.zeros(8, dtype=torch.int32, device=dev)
    p = one.data_ptr()
    rc = L.fo_decode_sparse_static(None, None, None, None, p, p, p, limit // 8 + 1, 8, 128, 1, p, p, p, p, p, p, p, p,
                                   None, torch.cuda.current_stream(dev).cuda_stream)
    assert rc == -1 and b"built-in scratch" in L.fo_last_error()


def test_static_scratch_decoder_in_a_captured_graph(dev):
    """The entry point is meant for callers that cannot allocate, a captured HIP graph among them.  Its
    first call on a device looks up the address of the built-in array (not a stream operation): that
    call is made eagerly here, as the header asks, and the capture follows.  The graph is replayed
    three times with eager work and synchronisations in between, on symbols rewritten in place between
    the replays; every replay must give what fo_decode_sparse gives for the symbols of that moment."""
    from flashomni_amd import _lib
    L = _lib.lib()
    heads, ql, kl = 6, [700, 129], [640, 300]
    masks = [make_ragged_masks(ql, kl, heads, 0.7, pk, seed=60 + i) for i, pk in enumerate((0.4, 0.8))]
    qo, kv = torch.from_numpy(masks[0]["qo_indptr"]), torch.from_numpy(masks[0]["kv_indptr"])
    sizes = torch.zeros(3, dtype=torch.int64)
    _lib.check(L.fo_decode_sizes(qo.data_ptr(), kv.data_ptr(), 2, heads, 128, 128, sizes[0:].data_ptr(),
                                 sizes[1:].data_ptr(), sizes[2:].data_ptr()))
    n_blk, max_rows, max_nnz = (int(v) for v in sizes)
    table = torch.empty((2, n_blk), dtype=torch.int32)
    _lib.check(L.fo_sparse_block_table(qo.data_ptr(), 2, 128, table[0].data_ptr(), table[1].data_ptr(), n_blk,
                                       sizes[0:].data_ptr()))
    table_d, kv_d = table.to(dev), kv.to(dev)
    t = lambda a: torch.from_numpy(a).to(dev)
    sym = [t(masks[0][n]) for n in ("packed_info", "packed_keep", "info_indptr", "keep_indptr")]
    b = _buffers(dev, max_rows, max_nnz)
    head = [s.data_ptr() for s in sym] + [table_d[0].data_ptr(), table_d[1].data_ptr(), kv_d.data_ptr(), n_blk,
                                          heads, 128, 0]
    names = ("row_req", "row_qb", "row_head", "kv_row_ptr", "kv_idx", "counts", "order", "sched")
    outs = [b[n].data_ptr() for n in names]

    def static_call():
        _lib.check(L.fo_decode_sparse_static(*head, *outs, b["shares"].data_ptr(),
                                             torch.cuda.current_stream(dev).cuda_stream))

    static_call()   # eager first call: resolves the array's address on this device
    torch.cuda.synchronize(dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_call()
    for which in (1, 0, 1):
        for s, n in zip(sym, ("packed_info", "packed_keep", "info_indptr", "keep_indptr")):
            s.copy_(t(masks[which][n]))
        for n in names + ("shares",):
            b[n].fill_(-7)
        torch.cuda.synchronize(dev)
        graph.replay()
        torch.cuda.synchronize(dev)
        got = {k: v.cpu().numpy() for k, v in b.items()}
        exp, _ = _decode(dev, masks[which], heads, False, True)
        assert _assert_same(got, exp) > 0
