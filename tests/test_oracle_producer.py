"""Pins oracle/producer.py (scores -> symbols) without a GPU: hand-worked rows, a brute force that
removes the smallest entry one at a time, the reference script's own consistency checks
(benchmark/test_attn_score.py:155-160) and mass invariants."""
import numpy as np
import pytest

from oracle import producer, symbols


def _scores_with_probs(probs):
    """Scores whose softmax is `probs` (up to fp32 rounding of log/exp)."""
    return np.log(np.asarray(probs, dtype=np.float64)).astype(np.float32)


def test_hand_worked_kv_row():
    # probabilities 0.4 0.1 0.3 0.2 ; ascending: idx1 (.1) idx3 (.2) idx2 (.3) idx0 (.4); cdf .1 .3 .6 1
    row = _scores_with_probs([0.4, 0.1, 0.3, 0.2])
    pooled = np.zeros((1, 1, 2, 4), dtype=np.float32)
    pooled[0, 0, 1] = row
    for thr, expect in [(0.05, [1, 1, 1, 1]), (0.15, [1, 0, 1, 1]), (0.35, [1, 0, 1, 0]),
                        (0.65, [1, 0, 0, 0]), (1.5, [0, 0, 0, 0])]:
        kv = producer.kv_symbols(pooled, 1, [thr])
        assert kv[0, 0, 0].tolist() == [1, 1, 1, 1]          # text row keeps everything
        assert kv[0, 0, 1].tolist() == expect, thr


def test_hand_worked_q_symbols_sum_over_heads_and_text_rows():
    # two heads, two text q blocks, NQ = NK = 5, three image key blocks.
    # the four contributing rows add up to log-probabilities of (0.5, 0.125, 0.375)
    target = np.log(np.array([0.5, 0.125, 0.375]))
    pooled = np.random.default_rng(0).normal(size=(1, 2, 5, 5)).astype(np.float32)
    pooled[0, :, :2, 2:] = (target / 4).astype(np.float32)
    si = producer.q_symbols(pooled, 2, 2, [0.2])
    # only the 0.125 block fits 0.2; it is image block 1 -> q block 2 + 1, for both heads
    assert si.tolist() == [[[1, 1, 1, 0, 1], [1, 1, 1, 0, 1]]]
    si = producer.q_symbols(pooled, 2, 2, [0.51])
    assert si.tolist() == [[[1, 1, 1, 0, 0], [1, 1, 1, 0, 0]]]
    si = producer.q_symbols(pooled, 2, 2, [0.1])
    assert si.min() == 1


def _brute_force_drop(row, thr):
    """Remove the smallest remaining entry (lowest index on ties) while the removed mass fits."""
    x = np.asarray(row, dtype=np.float64)
    p = np.exp(x - x.max())
    p /= p.sum()
    alive = list(range(len(x)))
    dropped, mass = [], 0.0
    while alive:
        j = min(alive, key=lambda i: (row[i], i))
        if mass + p[j] > thr:
            break
        mass += p[j]
        dropped.append(j)
        alive.remove(j)
    return sorted(dropped)


@pytest.mark.parametrize("seed", range(6))
def test_kv_symbols_match_brute_force(seed):
    rng = np.random.default_rng(seed)
    B, H, NQ, NK, t2t = 2, 3, 6, 9, 2
    pooled = rng.normal(scale=2.0, size=(B, H, NQ, NK)).astype(np.float32)
    thr = rng.uniform(0.05, 0.6, size=H).astype(np.float32)
    kv = producer.kv_symbols(pooled, t2t, thr)
    lo, hi = producer.selection_bounds(pooled, thr.reshape(1, H, 1))
    assert (kv[:, :, :t2t] == 1).all()
    for b in range(B):
        for h in range(H):
            for q in range(t2t, NQ):
                if lo[b, h, q] != hi[b, h, q]:
                    continue        # mass within rounding of the threshold: not a fair row
                want = _brute_force_drop(pooled[b, h, q], float(thr[h]))
                got = np.nonzero(kv[b, h, q] == 0)[0].tolist()
                assert got == want, (b, h, q)


def test_equal_scores_are_taken_in_index_order():
    pooled = np.zeros((1, 1, 1, 8), dtype=np.float32)       # eight equal scores, 1/8 each
    kv = producer.kv_symbols(pooled, 0, [0.3])              # two fit (0.25), three do not
    assert kv[0, 0, 0].tolist() == [0, 0, 1, 1, 1, 1, 1, 1]


def test_joint_fill_equals_separate_fills():
    """What the reference script prints at benchmark/test_attn_score.py:155-160."""
    rng = np.random.default_rng(3)
    B, H, N, t2t = 2, 2, 5, 2
    pooled = rng.normal(size=(B, H, N, N)).astype(np.float32)
    t2i = pooled[:, :, :t2t, t2t:].sum(axis=(1, 2), dtype=np.float32)
    q_order = producer.ascending_order(t2i)
    q_sel = producer.num_to_select(producer.softmax_f32(t2i), q_order, np.full(B, 0.2))
    ones_q = np.ones((B, H, N), dtype=np.uint8)
    ones_kv = np.ones((B, H, N, N), dtype=np.uint8)
    si = producer.fill_sparse_info(ones_q, q_sel, q_order, t2t)

    img = pooled[:, :, t2t:, :]
    order = producer.ascending_order(img)
    sel = producer.num_to_select(producer.softmax_f32(img), order, np.full((B, H, N - t2t), 0.2))
    kv = producer.fill_sparse_kv_info(ones_kv, sel, order, t2t)

    order_all = producer.ascending_order(pooled)
    sel_all = producer.num_to_select(producer.softmax_f32(pooled), order_all, np.full((B, H, N), 0.2))
    kv_all, si_all = producer.fill_flashomni(ones_kv, sel_all, order_all, ones_q, q_sel, q_order, t2t)
    assert np.array_equal(si, si_all)
    assert np.array_equal(kv, kv_all)
    assert (kv[:, :, :t2t] == 1).all()
    # and the one-call forms agree with the step-by-step ones
    assert np.array_equal(si, producer.q_symbols(pooled, t2t, t2t, np.full(B, 0.2)))
    assert np.array_equal(kv, producer.kv_symbols(pooled, t2t, np.full(H, 0.2)))


def test_mass_invariants():
    rng = np.random.default_rng(5)
    B, H, NQ, NK, t2t = 1, 4, 12, 40, 3
    pooled = rng.normal(scale=1.5, size=(B, H, NQ, NK)).astype(np.float32)
    thr = np.array([0.0, 0.1, 0.5, 0.9], dtype=np.float32)
    kv = producer.kv_symbols(pooled, t2t, thr)
    p = producer.softmax_f32(pooled).astype(np.float64)
    for h in range(H):
        for q in range(t2t, NQ):
            dropped = kv[0, h, q] == 0
            mass = p[0, h, q][dropped].sum()
            assert mass <= thr[h] + 1e-5
            if (~dropped).any():
                # the next candidate does not fit, and nothing kept scores below something dropped
                assert mass + p[0, h, q][~dropped].min() > thr[h] - 1e-5
                if dropped.any():
                    assert pooled[0, h, q][dropped].max() <= pooled[0, h, q][~dropped].min()
    assert (kv[0, 0] == 1).all()        # threshold 0 drops nothing


def test_kernel_layout_bits():
    rng = np.random.default_rng(7)
    B, H, NQ, NK = 2, 3, 4, 5
    si = (rng.random((B, H, NQ)) < 0.5).astype(np.uint8)
    kv = (rng.random((B, H, NQ, NK)) < 0.5).astype(np.uint8)
    flat_si, flat_kv = producer.to_kernel_layout(si, kv)
    for b in range(B):
        packed_si = symbols.packbits(flat_si[b], "little")
        packed_kv = symbols.packbits(flat_kv[b], "little")
        for q in range(NQ):
            for h in range(H):
                assert symbols.get_bit(packed_si, 0, q * H + h) == si[b, h, q]
                for k in range(NK):
                    assert symbols.get_bit(packed_kv, 0, (q * H + h) * NK + k) == kv[b, h, q, k]
