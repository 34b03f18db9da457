"""GPU parity: packbits / segment_packbits / sparse-symbol decoder vs the oracle (bit-exact)."""
import numpy as np
import pytest
import torch

import oracle
from helpers import make_ragged_masks

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [0, 1, 7, 8, 9, 64, 1000, 31104, 1 << 20])
@pytest.mark.parametrize("bitorder", ["big", "little"])
def test_packbits_matches_oracle(dev, n, bitorder):
    import flashomni_amd as fo
    rng = np.random.default_rng(n + 1)
    x = rng.random(n) < 0.5
    y = fo.packbits(torch.from_numpy(x).to(dev), bitorder)
    assert y.dtype == torch.uint8 and y.numel() == (n + 7) // 8
    np.testing.assert_array_equal(y.cpu().numpy(), oracle.packbits(x, bitorder))


def test_packbits_docstring_vectors(dev):
    import flashomni_amd as fo
    x = torch.tensor([1, 0, 1, 1, 0, 0, 1, 1], dtype=torch.bool, device=dev)
    assert fo.packbits(x).tolist() == [0b10110011]
    x = torch.tensor([1, 0, 1, 1, 0, 0, 1, 1, 1, 0, 1], dtype=torch.bool, device=dev)
    y, p = fo.segment_packbits(x, torch.tensor([0, 4, 7, 11], device=dev), bitorder="big")
    assert y.tolist() == [0b10110000, 0b100000, 0b11010000]
    assert p.tolist() == [0, 1, 2, 3]


def test_packbits_nonbool_input_and_bad_bitorder(dev):
    import flashomni_amd as fo
    x = torch.tensor([3, 0, 255, 0, 0, 0, 0, 1, 2], dtype=torch.uint8, device=dev)
    assert fo.packbits(x, "little").tolist() == [0b10000101, 0b1]
    with pytest.raises(RuntimeError, match="bitorder must be 'big' or 'little'"):
        fo.packbits(x, "middle")


@pytest.mark.parametrize("bitorder", ["big", "little"])
def test_segment_packbits_ragged(dev, bitorder):
    import flashomni_amd as fo
    rng = np.random.default_rng(5)
    lens = [0, 1, 8, 13, 4000, 0, 77, 31104]
    indptr = np.zeros(len(lens) + 1, dtype=np.int32)
    indptr[1:] = np.cumsum(lens)
    x = rng.random(indptr[-1]) < 0.4
    y, p = fo.segment_packbits(torch.from_numpy(x).to(dev), torch.from_numpy(indptr).to(dev), bitorder)
    ey, ep = oracle.segment_packbits(x, indptr, bitorder)
    np.testing.assert_array_equal(p.cpu().numpy(), ep)
    np.testing.assert_array_equal(y.cpu().numpy(), ey)


def _decode_on_gpu(dev, m, heads, is_full=False):
    import flashomni_amd as fo
    ws = torch.empty(128 << 20, dtype=torch.uint8, device=dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(ws)
    w.plan(torch.from_numpy(m["qo_indptr"]), torch.from_numpy(m["kv_indptr"]), heads, heads, 128,
           q_data_type=torch.bfloat16)
    t = lambda a: torch.from_numpy(a).to(dev)
    wl = w.decode(t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]),
                  is_full)
    return [a.numpy() for a in wl.to_host()]


CASES = [
    ([4608], [4608], 24, 0.75, 0.5),                 # FLUX shape
    ([300, 1, 128, 1000], [77, 513, 128, 4096], 3, 0.6, 0.3),   # ragged, NKV not multiple of 8
    ([129], [128 * 67 + 5], 5, 0.9, 0.02),           # long rows crossing many bytes
    ([256, 256], [256, 256], 1, 0.5, 0.5),
    ([200, 0, 128, 1], [300, 64, 0, 5], 3, 0.8, 0.6),           # a request without q rows, one without keys
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("force", [None, "ones", "zeros"])
def test_decoder_matches_bruteforce(dev, case, force):
    ql, kl, heads, pa, pk = case
    m = make_ragged_masks(ql, kl, heads, pa, pk, seed=len(ql) + heads, force=force)
    got = _decode_on_gpu(dev, m, heads)
    exp = oracle.decode_kv_csr(m["packed_info"], m["packed_keep"], m["info_indptr"],
                               m["keep_indptr"], m["qo_indptr"], m["kv_indptr"], heads, 128, 128)
    for g, e, name in zip(got, exp, ["row_req", "row_qb", "row_head", "kv_row_ptr", "kv_idx"]):
        np.testing.assert_array_equal(g, e, err_msg=name)


def test_decoder_is_full_lists_everything(dev):
    ql, kl, heads = [300, 128], [500, 64], 2
    m = make_ragged_masks(ql, kl, heads, 0.5, 0.5, seed=3)
    got = _decode_on_gpu(dev, m, heads, is_full=True)
    exp = oracle.decode_kv_csr(None, None, None, None, m["qo_indptr"], m["kv_indptr"], heads, 128, 128,
                               is_full=True)
    for g, e in zip(got, exp):
        np.testing.assert_array_equal(g, e)


@pytest.mark.parametrize("index", [3, 4])
def test_decoder_full_size_configs(dev, index):
    """Hunyuan / Wan shaped masks at full size: bit-exact against the brute-force enumeration."""
    from flashomni_amd.workloads import make_workload
    wl = make_workload(index, tensors=False)
    m = dict(packed_info=wl.packed_info.numpy(), packed_keep=wl.packed_kv_info.numpy(),
             info_indptr=wl.info_indptr.numpy(), keep_indptr=wl.kv_info_indptr.numpy(),
             qo_indptr=wl.qo_indptr.numpy(), kv_indptr=wl.kv_indptr.numpy())
    got = _decode_on_gpu(dev, m, wl.shape.heads)
    exp = oracle.decode_kv_csr(m["packed_info"], m["packed_keep"], m["info_indptr"], m["keep_indptr"],
                               m["qo_indptr"], m["kv_indptr"], wl.shape.heads, 128, 128)
    for g, e in zip(got, exp):
        np.testing.assert_array_equal(g, e)
    assert len(got[0]) == wl.active_rows and len(got[4]) == wl.computed_blocks


@pytest.mark.parametrize("case", CASES[:3])
def test_decoder_execution_order(dev, case):
    """`order` / `sched`: a permutation of the rows, cut into 8 queues by head % 8, heads back to
    back inside a queue, and inside a head no row is followed by one of a longer length class."""
    import flashomni_amd as fo
    ql, kl, heads, pa, pk = case
    m = make_ragged_masks(ql, kl, heads, pa, pk, seed=7)
    ws = torch.empty(128 << 20, dtype=torch.uint8, device=dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(ws)
    w._share_rows = False                       # whole rows from the queues
    w.plan(torch.from_numpy(m["qo_indptr"]), torch.from_numpy(m["kv_indptr"]), heads, heads, 128,
           q_data_type=torch.bfloat16)
    t = lambda a: torch.from_numpy(a).to(dev)
    wl = w.decode(t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]))
    n_rows, _ = wl.sizes()
    order = wl.order[:n_rows].cpu().numpy()
    sched = wl.sched.cpu().numpy()
    row_head = wl.row_head[:n_rows].cpu().numpy()
    ptr = wl.kv_row_ptr[:n_rows + 1].cpu().numpy()
    lens = ptr[1:] - ptr[:-1]
    assert sorted(order.tolist()) == list(range(n_rows))
    assert sched[0] == 0 and sched[8] == n_rows and (sched[16:25] == 0).all() and sched[26] == 0
    max_n = int(lens.max()) if n_rows else 0
    assert sched[25] == max_n
    n_classes = min(32, 8192 // heads)
    for x in range(8):
        seg = order[sched[x]:sched[x + 1]]
        h = row_head[seg]
        assert (h % 8 == x).all()
        assert (np.diff(h) >= 0).all()          # heads back to back, ascending
        cls = (max_n - lens[seg]).astype(np.int64) * n_classes // (max_n + 1)
        same_head = np.diff(h) == 0
        assert (np.diff(cls)[same_head] >= 0).all()   # longest class first inside a head


@pytest.mark.parametrize("case", [([2304], [2304], 24, 0.75, 0.5)] + CASES[1:])
def test_decoder_even_shares(dev, case):
    """Few rows per CU: `order` lists the rows head by head in canonical order, a row costs
    3 + its kv blocks, and the share table cuts the cost line into one range per CU."""
    import flashomni_amd as fo
    ql, kl, heads, pa, pk = case
    m = make_ragged_masks(ql, kl, heads, pa, pk, seed=7)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w.plan(torch.from_numpy(m["qo_indptr"]), torch.from_numpy(m["kv_indptr"]), heads, heads, 128,
           q_data_type=torch.bfloat16)
    t = lambda a: torch.from_numpy(a).to(dev)
    wl = w.decode(t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]))
    n_rows, _ = wl.sizes()
    n_cu = torch.cuda.get_device_properties(dev).multi_processor_count
    assert 0 < n_rows <= 2 * n_cu
    sched = wl.sched.cpu().numpy()
    order = wl.order[:n_rows].cpu().numpy()
    shares = wl.shares.cpu().numpy()
    row_head = wl.row_head[:n_rows].cpu().numpy()
    ptr = wl.kv_row_ptr[:n_rows + 1].cpu().numpy()
    lens = (ptr[1:] - ptr[:-1]).astype(np.int64)
    exp_order = np.argsort(row_head, kind="stable")
    assert (order == exp_order).all()
    cost = 3 + lens[exp_order]
    start = np.concatenate([[0], np.cumsum(cost)])[:-1] + 3
    total = int(cost.sum())
    assert (shares[512:512 + n_rows] == start).all() and shares[512 + n_rows] == total + 3
    max_n = int(lens.max())
    share = max(-(-total // n_cu), (max_n + 2) // 3, 1)
    assert list(sched[25:31]) == [max_n, 1, share, total, n_cu, n_rows]
    assert (sched[16:25] == 0).all() and (sched[64:576] == 0).all()
    assert [int(sched[x]) for x in range(9)] == [n_rows * x // 8 for x in range(9)]
    end = start + lens[exp_order]
    for j in range(n_cu):
        first = int(np.searchsorted(end, j * share, side="right"))   # first row with end > j * share
        assert shares[j] == first, j
    # a row touches at most four shares
    touched = (end - 1) // share - np.minimum(start, end - 1) // share + 1
    assert touched.max() <= 4


def test_decoder_queue_records(dev):
    """More than two rows per CU and a share table: the queues are laid out as without one, and the
    table holds one record per queue entry (row, request, q block, head, first kv slot, kv count)."""
    import flashomni_amd as fo
    ql, kl, heads, pa, pk = [4608, 1000], [4608, 700], 24, 0.75, 0.5
    m = make_ragged_masks(ql, kl, heads, pa, pk, seed=7)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w.plan(torch.from_numpy(m["qo_indptr"]), torch.from_numpy(m["kv_indptr"]), heads, heads, 128,
           q_data_type=torch.bfloat16)
    t = lambda a: torch.from_numpy(a).to(dev)
    wl = w.decode(t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]))
    n_rows, _ = wl.sizes()
    n_cu = torch.cuda.get_device_properties(dev).multi_processor_count
    assert n_rows > 2 * n_cu
    sched = wl.sched.cpu().numpy()
    assert sched[26] == 0 and sched[31] == 1 and sched[8] == n_rows
    order = wl.order[:n_rows].cpu().numpy()
    rec = wl.shares.cpu().numpy()[512:512 + 8 * n_rows].reshape(n_rows, 8)
    ptr = wl.kv_row_ptr[:n_rows + 1].cpu().numpy()
    assert sorted(order.tolist()) == list(range(n_rows))
    assert (rec[:, 0] == order).all()
    assert (rec[:, 1] == wl.row_req[:n_rows].cpu().numpy()[order]).all()
    assert (rec[:, 2] == wl.row_qb[:n_rows].cpu().numpy()[order]).all()
    assert (rec[:, 3] == wl.row_head[:n_rows].cpu().numpy()[order]).all()
    assert (rec[:, 4] == ptr[order]).all() and (rec[:, 5] == ptr[order + 1] - ptr[order]).all()


@pytest.mark.parametrize("share_table", [True, False])
def test_decoder_long_list_order(dev, share_table):
    """Eight or more rows per CU: inside a head the rows are queued with ascending (request, q block),
    a fixed order; queues by head % 8; with a share table one record per queue entry."""
    import flashomni_amd as fo
    n_cu = torch.cuda.get_device_properties(dev).multi_processor_count
    heads = 12
    nq = -(-(8 * n_cu) // heads) + 40           # enough q blocks for 8 rows per CU at p = 0.9
    ql, kl = [nq * 128 - 50, 700], [1500, 300]
    m = make_ragged_masks(ql, kl, heads, 0.9, 0.5, seed=9)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w._share_rows = share_table
    w.plan(torch.from_numpy(m["qo_indptr"]), torch.from_numpy(m["kv_indptr"]), heads, heads, 128,
           q_data_type=torch.bfloat16)
    t = lambda a: torch.from_numpy(a).to(dev)
    wl = w.decode(t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]))
    n_rows, _ = wl.sizes()
    assert n_rows >= 8 * n_cu
    sched = wl.sched.cpu().numpy()
    order = wl.order[:n_rows].cpu().numpy()
    row_head = wl.row_head[:n_rows].cpu().numpy()
    ptr = wl.kv_row_ptr[:n_rows + 1].cpu().numpy()
    # canonical positions ascend with (request, q block): a head's rows in canonical order
    exp = np.concatenate([np.nonzero(row_head == h)[0] for x in range(8) for h in range(x, heads, 8)])
    assert (order == exp).all()
    bounds = np.concatenate([[0], np.cumsum([sum(int((row_head == h).sum()) for h in range(x, heads, 8))
                                             for x in range(8)])])
    assert (sched[:9] == bounds).all()
    assert (sched[16:25] == 0).all() and sched[25] == int((ptr[1:] - ptr[:-1]).max())
    assert sched[26] == 0 and sched[31] == int(share_table) and sched[32] == 1
    if share_table:
        rec = wl.shares.cpu().numpy()[512:512 + 8 * n_rows].reshape(n_rows, 8)
        assert (rec[:, 0] == order).all()
        assert (rec[:, 1] == wl.row_req[:n_rows].cpu().numpy()[order]).all()
        assert (rec[:, 2] == wl.row_qb[:n_rows].cpu().numpy()[order]).all()
        assert (rec[:, 3] == row_head[order]).all()
        assert (rec[:, 4] == ptr[order]).all() and (rec[:, 5] == ptr[order + 1] - ptr[order]).all()
        assert (rec[:, 6:] == 0).all()
