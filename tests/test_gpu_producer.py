"""GPU parity: symbol producer (pooled scores -> packed sparse_info / sparse_kv_info) vs the oracle.

The dropped entries of a row must be exactly the n lowest in (score, index) order.  n must equal the
oracle's count, except for rows whose cumulative probability comes within 1e-5 of the threshold
(the reference's own fp32 cumulative sum is not specified to better than that): there n may be any
count the fp64 bounds admit.  The bit layout of the packed outputs is checked bit-exactly."""
import numpy as np
import pytest
import torch

import oracle
from oracle import producer

pytestmark = pytest.mark.gpu

EPS = 1e-5


def _unpack(outputs, B, H, NQ, NK):
    """Packed GPU outputs -> uint8 maps [B, H, NQ], [B, H, NQ, NK]; checks indptrs and padding."""
    si, si_ip, kv, kv_ip = [t.cpu().numpy() for t in outputs]
    si_bytes, kv_bytes = (NQ * H + 7) // 8, (NQ * H * NK + 7) // 8
    np.testing.assert_array_equal(si_ip, np.arange(B + 1, dtype=np.int64) * si_bytes)
    np.testing.assert_array_equal(kv_ip, np.arange(B + 1, dtype=np.int64) * kv_bytes)
    assert si.dtype == np.uint8 and si.size == B * si_bytes and kv.size == B * kv_bytes
    maps_q = np.zeros((B, H, NQ), dtype=np.uint8)
    maps_kv = np.zeros((B, H, NQ, NK), dtype=np.uint8)
    for b in range(B):
        bits = np.unpackbits(si[b * si_bytes:(b + 1) * si_bytes], bitorder="little")
        assert not bits[NQ * H:].any(), "padding bits of sparse_info must be zero"
        maps_q[b] = bits[:NQ * H].reshape(NQ, H).T
        bits = np.unpackbits(kv[b * kv_bytes:(b + 1) * kv_bytes], bitorder="little")
        assert not bits[NQ * H * NK:].any(), "padding bits of sparse_kv_info must be zero"
        maps_kv[b] = bits[:NQ * H * NK].reshape(NQ, H, NK).transpose(1, 0, 2)
    return maps_q, maps_kv


def _check_rows(scores, thr, dropped, expect_dropped):
    """scores [R, n] fp32, thr [R], dropped / expect_dropped [R, n] bool.  Returns the number of
    rows on which the two counts differ (all of them within the admissible interval)."""
    lo, hi = producer.selection_bounds(scores, thr, EPS)
    order = producer.ascending_order(scores)
    rank = np.argsort(order, axis=-1, kind="stable")
    n = dropped.sum(axis=-1)
    assert ((lo <= n) & (n <= hi)).all(), "count outside the admissible interval"
    np.testing.assert_array_equal(dropped, rank < n[:, None], err_msg="not the n lowest entries")
    firm = lo == hi
    np.testing.assert_array_equal(dropped[firm], expect_dropped[firm])
    return int((n != expect_dropped.sum(axis=-1)).sum())


def _run_case(dev, B, H, NQ, NK, t2t, q_thr, kv_thr, dtype=torch.float32, seed=0, scale=1.5,
              integer_scores=False):
    import flashomni_amd as fo
    rng = np.random.default_rng(seed)
    pooled = rng.normal(scale=scale, size=(B, H, NQ, NK)).astype(np.float32)
    if integer_scores:
        pooled = np.round(pooled)                # many equal scores
    t = torch.from_numpy(pooled).to(dtype)
    pooled = t.float().numpy()                   # what the kernel sees
    q_thr = np.broadcast_to(np.asarray(q_thr, dtype=np.float32), (B,)).copy()
    kv_thr = np.broadcast_to(np.asarray(kv_thr, dtype=np.float32), (H,)).copy()
    out = fo.sparse_symbols_from_scores(t.to(dev), t2t, torch.from_numpy(q_thr).to(dev),
                                        torch.from_numpy(kv_thr).to(dev))
    got_q, got_kv = _unpack(out, B, H, NQ, NK)

    # kv symbols
    exp_kv = producer.kv_symbols(pooled, t2t, kv_thr)
    assert (got_kv[:, :, :t2t] == 1).all(), "text q rows keep every key block"
    rows = pooled[:, :, t2t:, :].reshape(-1, NK)
    thr_rows = np.broadcast_to(kv_thr.reshape(1, H, 1), (B, H, NQ - t2t)).reshape(-1)
    moved = _check_rows(rows, thr_rows, got_kv[:, :, t2t:].reshape(-1, NK) == 0,
                        exp_kv[:, :, t2t:].reshape(-1, NK) == 0)
    assert moved <= max(1, rows.shape[0] // 200)

    # q symbols: identical for every head, text q blocks never cached
    exp_q = producer.q_symbols(pooled, t2t, t2t, q_thr)
    assert (got_q == got_q[:, :1]).all()
    assert (got_q[:, :, :t2t] == 1).all()
    t2i = pooled[:, :, :t2t, t2t:].sum(axis=(1, 2), dtype=np.float32)
    n_img = NK - t2t
    if not integer_scores:       # summed scores differ by rounding between the two summation orders
        _check_rows(t2i, q_thr, got_q[:, 0, t2t:t2t + n_img] == 0, exp_q[:, 0, t2t:t2t + n_img] == 0)
    return out, got_q, got_kv


@pytest.mark.parametrize("shape", [
    (2, 3, 7, 7, 2),          # one slot per lane
    (1, 2, 70, 70, 4),        # two slots
    (2, 5, 200, 200, 4),      # four
    (1, 5, 595, 595, 4),      # ten: the Wan block count, 595 not a multiple of 8
    (1, 2, 1100, 1100, 8),    # twenty-four
    (1, 3, 36, 36, 4),        # the FLUX block count
])
def test_symbols_match_oracle(dev, shape):
    B, H, NQ, NK, t2t = shape
    kv_thr = np.linspace(0.05, 0.45, H)
    q_thr = np.linspace(0.1, 0.3, B)
    _run_case(dev, B, H, NQ, NK, t2t, q_thr, kv_thr, seed=NQ)


def test_largest_row_length(dev):
    _run_case(dev, 1, 1, 4096, 4096, 4, 0.2, 0.3, seed=9)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_half_precision_scores_have_equal_entries(dev, dtype):
    """16-bit scores repeat values inside a row: equal scores are taken in index order."""
    _run_case(dev, 1, 4, 300, 300, 4, 0.2, [0.1, 0.2, 0.3, 0.4], dtype=dtype, seed=11)


def test_many_equal_scores(dev):
    _run_case(dev, 2, 3, 130, 130, 2, 0.25, 0.35, seed=13, integer_scores=True)


def test_threshold_extremes(dev):
    B, H, NQ, NK, t2t = 1, 2, 40, 40, 3
    _, got_q, got_kv = _run_case(dev, B, H, NQ, NK, t2t, 0.0, [0.0, 1.5], seed=17)
    assert (got_kv[0, 0] == 1).all()                     # nothing fits a zero budget
    assert (got_kv[0, 1, t2t:] == 0).all()               # everything fits a budget above one
    assert (got_q == 1).all()


def test_no_text_blocks(dev):
    """T2T = 0: the q score is an empty sum, every image block equally likely, taken in index order."""
    import flashomni_amd as fo
    B, H, N = 1, 2, 16
    pooled = torch.randn(B, H, N, N, generator=torch.Generator().manual_seed(3))
    out = fo.sparse_symbols_from_scores(pooled.to(dev), 0, 0.26, 0.2)
    got_q, got_kv = _unpack(out, B, H, N, N)
    assert got_q[0, 0].tolist() == [0] * 4 + [1] * 12    # 4/16 = 0.25 fits, 5/16 does not
    exp_kv = producer.kv_symbols(pooled.numpy(), 0, np.full(H, 0.2, dtype=np.float32))
    np.testing.assert_array_equal(got_kv, exp_kv)


def test_symbols_feed_the_decoder(dev):
    """The packed output is what run()/decode() read: decoding it lists the kept blocks."""
    import flashomni_amd as fo
    B, H, N, t2t = 2, 3, 20, 4
    out, got_q, got_kv = _run_case(dev, B, H, N, N, t2t, 0.3, 0.4, seed=21)
    ws = torch.empty(32 << 20, dtype=torch.uint8, device=dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(ws)
    indptr = torch.arange(B + 1, dtype=torch.int32) * (N * 128)
    w.plan(indptr, indptr, H, H, 128, q_data_type=torch.bfloat16)
    wl = w.decode(out[0], out[2], out[1], out[3])
    row_req, row_qb, row_head, kv_row_ptr, kv_idx = [a.numpy() for a in wl.to_host()]
    flat_q, flat_kv = producer.to_kernel_layout(got_q, got_kv)
    exp = oracle.decode_kv_csr(
        np.concatenate([oracle.packbits(flat_q[b], "little") for b in range(B)]),
        np.concatenate([oracle.packbits(flat_kv[b], "little") for b in range(B)]),
        out[1].cpu().numpy(), out[3].cpu().numpy(), indptr.numpy(), indptr.numpy(), H, 128, 128)
    for g, e in zip((row_req, row_qb, row_head, kv_row_ptr, kv_idx), exp):
        np.testing.assert_array_equal(g, e)
    assert len(row_req) == int(got_q.sum())


def test_wan_size_properties(dev):
    """Full Wan block grid (40 heads, 595 x 595 blocks): size-independent properties on the GPU,
    and a sample of rows against the oracle."""
    import flashomni_amd as fo
    B, H, N, t2t = 1, 40, 595, 4
    g = torch.Generator().manual_seed(1004)
    pooled = (torch.randn(B, H, N, N, generator=g) * 2.0)
    kv_thr = torch.linspace(0.05, 0.5, H)
    out = fo.sparse_symbols_from_scores(pooled.to(dev), t2t, 0.2, kv_thr.to(dev))
    got_q, got_kv = _unpack(out, B, H, N, N)
    dropped = torch.from_numpy(got_kv[0] == 0).to(dev)                 # [H, N, N]
    s = pooled[0].to(dev).double()
    p = torch.softmax(s, dim=-1)
    mass = (p * dropped).sum(-1)                                       # [H, N]
    thr = kv_thr.to(dev).double()[:, None]
    assert bool((mass[:, t2t:] <= thr + EPS).all())
    assert not bool(dropped[:, :t2t].any())
    kept_min_p = torch.where(dropped, torch.full_like(p, 2.0), p).amin(-1)
    assert bool((mass + kept_min_p > thr - EPS)[:, t2t:].all()), "a further block would have fitted"
    drop_max = torch.where(dropped, s, torch.full_like(s, -1e30)).amax(-1)
    kept_min = torch.where(dropped, torch.full_like(s, 1e30), s).amin(-1)
    assert bool((drop_max <= kept_min).all()), "a kept block scores below a dropped one"
    # sample of rows against the oracle
    rng = np.random.default_rng(0)
    hs, qs = rng.integers(0, H, 64), rng.integers(t2t, N, 64)
    rows = pooled[0].numpy()[hs, qs]
    sample = np.zeros((1, 1, 64, N), dtype=np.float32)
    sample[0, 0] = rows
    for i in range(64):
        exp = producer.kv_symbols(sample[:, :, i:i + 1], 0, [float(kv_thr[hs[i]])])[0, 0, 0]
        lo, hi = producer.selection_bounds(rows[i], float(kv_thr[hs[i]]), EPS)
        if lo == hi:
            np.testing.assert_array_equal(got_kv[0, hs[i], qs[i]], exp)


def test_argument_errors(dev):
    import flashomni_amd as fo
    x = torch.zeros(1, 2, 8, 8, device=dev)
    with pytest.raises(ValueError, match=r"\[B, H, NQ, NK\]"):
        fo.sparse_symbols_from_scores(x[0], 2, 0.2, 0.2)
    with pytest.raises(ValueError, match="kv_threshold must have 2 entries"):
        fo.sparse_symbols_from_scores(x, 2, 0.2, torch.zeros(3))
    with pytest.raises(RuntimeError, match="text blocks"):
        fo.sparse_symbols_from_scores(x, 9, 0.2, 0.2)
    with pytest.raises(RuntimeError, match="do not fit behind"):
        fo.sparse_symbols_from_scores(x, 4, 0.2, 0.2, num_text_kv_blocks=2)
    with pytest.raises(ValueError, match="unsupported dtype"):
        fo.sparse_symbols_from_scores(x.double(), 2, 0.2, 0.2)
    with pytest.raises(ValueError):
        fo.sparse_symbols_from_scores(x.cpu(), 2, 0.2, 0.2)
