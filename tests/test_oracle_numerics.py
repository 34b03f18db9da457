"""CPU: the floating-point oracles pinned against library routines and closed forms
(dense attention -> torch SDPA, single-block softmax, permutation invariance; masked GEMMs ->
F.linear and the cache+final identity; fp8 quantiser -> torch's own e4m3fn cast)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from helpers import make_ragged_masks, sentinel_like


def _qkv(nq, nk, heads, seed):
    g = torch.Generator().manual_seed(seed)
    mk = lambda n: torch.randn(n, heads, 128, generator=g).to(torch.bfloat16)
    return mk(nq), mk(nk), mk(nk)


def test_attention_all_ones_equals_sdpa():
    heads = 2
    m = make_ragged_masks([200, 128], [300, 77], heads, force="ones")
    q, k, v = _qkv(328, 377, heads, 0)
    out = oracle.sparse_attention(q.float(), k.float(), v.float(), m["packed_info"], m["packed_keep"],
                                  m["info_indptr"], m["keep_indptr"], m["qo_indptr"], m["kv_indptr"])
    full = oracle.sparse_attention(q.float(), k.float(), v.float(), None, None, None, None,
                                   m["qo_indptr"], m["kv_indptr"], is_full=True)
    for (q0, q1), (k0, k1) in (((0, 200), (0, 300)), ((200, 328), (300, 377))):
        ref = F.scaled_dot_product_attention(q[q0:q1].float().transpose(0, 1), k[k0:k1].float().transpose(0, 1),
                                             v[k0:k1].float().transpose(0, 1)).transpose(0, 1)
        assert torch.allclose(out[q0:q1], ref, atol=2e-5, rtol=1e-4)
        assert torch.allclose(full[q0:q1], ref, atol=2e-5, rtol=1e-4)


def test_attention_block_mask_equals_sdpa_with_expanded_mask():
    """Same mask construction as benchmark/test_flashomni_attention.py:197-199."""
    heads, n = 3, 512
    m = make_ragged_masks([n], [n], heads, p_active=1.0, p_keep=0.5, seed=4)
    keep = m["keep"][0]
    keep[:, :, 0] = True   # SDPA needs at least one key per row
    m["packed_keep"] = np.packbits(keep.reshape(-1).astype(np.uint8), bitorder="little")
    q, k, v = _qkv(n, n, heads, 1)
    out = oracle.sparse_attention(q.float(), k.float(), v.float(), m["packed_info"], m["packed_keep"],
                                  m["info_indptr"], m["keep_indptr"], m["qo_indptr"], m["kv_indptr"])
    mask = torch.from_numpy(keep).permute(1, 0, 2)            # [H, NQ, NKV]
    mask = mask.repeat_interleave(128, 1).repeat_interleave(128, 2)[:, :n, :n]
    ref = F.scaled_dot_product_attention(q.float().transpose(0, 1), k.float().transpose(0, 1),
                                         v.float().transpose(0, 1), attn_mask=mask).transpose(0, 1)
    assert torch.allclose(out, ref, atol=2e-5, rtol=1e-4)


def test_attention_single_block_is_plain_softmax_and_lse_is_base2():
    heads = 1
    q, k, v = _qkv(128, 384, heads, 2)
    info = np.array([1], dtype=np.uint8)
    keep = np.packbits(np.array([0, 1, 0], dtype=np.uint8), bitorder="little")
    lse = torch.zeros(128, 1)
    out = oracle.sparse_attention(q.float(), k.float(), v.float(), info, keep, [0, 1], [0, 1], [0, 128], [0, 384],
                                  lse=lse)
    s = (q[:, 0].float() @ k[128:256, 0].float().T) / math.sqrt(128)
    ref = torch.softmax(s, -1) @ v[128:256, 0].float()
    assert torch.allclose(out[:, 0], ref, atol=2e-5, rtol=1e-4)
    assert torch.allclose(lse[:, 0], torch.logsumexp(s, -1) / math.log(2), atol=1e-4)


def test_attention_skipped_untouched_empty_zero_and_tail_crop():
    heads = 2
    q, k, v = _qkv(256, 200, heads, 3)
    # rows (qb,h): (0,0) active keep{1}, (0,1) cached, (1,0) active keep{}, (1,1) active keep{0,1}
    info = np.packbits(np.array([1, 0, 1, 1], dtype=np.uint8), bitorder="little")
    keep = np.packbits(np.array([0, 1, 1, 1, 0, 0, 1, 1], dtype=np.uint8), bitorder="little")
    out0 = torch.full((256, heads, 128), 9.0)
    lse = torch.full((256, heads), 123.0)
    out = oracle.sparse_attention(q.float(), k.float(), v.float(), info, keep, [0, 1], [0, 1], [0, 256], [0, 200],
                                  out=out0.clone(), lse=lse)
    assert torch.equal(out[:128, 1], out0[:128, 1]) and torch.equal(lse[:128, 1], torch.full((128,), 123.0))
    assert float(out[128:, 0].abs().max()) == 0.0 and torch.equal(lse[128:, 0], torch.full((128,), -5e4))
    # second kv block is cropped at kv_len = 200 (72 valid keys)
    s = (q[:128, 0].float() @ k[128:200, 0].float().T) / math.sqrt(128)
    assert torch.allclose(out[:128, 0], torch.softmax(s, -1) @ v[128:200, 0].float(), atol=2e-5, rtol=1e-4)


def test_attention_is_invariant_to_kv_block_permutation():
    heads = 1
    q, k, v = _qkv(128, 512, heads, 5)
    info = np.array([1], dtype=np.uint8)
    keep = np.packbits(np.array([1, 0, 1, 1], dtype=np.uint8), bitorder="little")
    a = oracle.sparse_attention(q.float(), k.float(), v.float(), info, keep, [0, 1], [0, 1], [0, 128], [0, 512])
    perm = torch.cat([torch.arange(384, 512), torch.arange(128, 256), torch.arange(256, 384), torch.arange(0, 128)])
    keep2 = np.packbits(np.array([1, 0, 1, 1], dtype=np.uint8)[[3, 1, 2, 0]], bitorder="little")
    b = oracle.sparse_attention(q.float(), k[perm].float(), v[perm].float(), info, keep2, [0, 1], [0, 1], [0, 128], [0, 512])
    assert torch.allclose(a, b, atol=1e-5)


def _flags(nq, heads, p, seed):
    rng = np.random.default_rng(seed)
    info = rng.random((nq, heads)) < p
    return info, np.packbits(info.reshape(-1).astype(np.uint8), bitorder="little")


def test_gemm_q_full_is_linear_and_skipped_tiles_keep_bytes():
    g = torch.Generator().manual_seed(0)
    x, w, b = torch.randn(1, 300, 96, generator=g), torch.randn(256, 96, generator=g), torch.randn(256, generator=g)
    full = oracle.gemm_q(x, w, 2, is_full=True, bias=b)
    assert torch.allclose(full, F.linear(x, w, b), atol=1e-5)
    info, packed = _flags(3, 2, 0.5, 1)
    out0 = torch.full((1, 300, 256), 5.0)
    out = oracle.gemm_q(x, w, 2, packed, [0, 1], 0, b, out=out0.clone())
    for iy in range(3):
        for ix in range(2):
            tile = (0, slice(iy * 128, min(300, iy * 128 + 128)), slice(ix * 128, ix * 128 + 128))
            if info[iy, ix]:
                assert torch.allclose(out[tile], F.linear(x, w, b)[tile], atol=1e-5)
            else:
                assert torch.equal(out[tile], out0[tile])
    # num_text_tokens shifts the q-block index (gemm.cuh:53)
    info2, packed2 = _flags(4, 2, 0.5, 2)
    out = oracle.gemm_q(x, w, 2, packed2, [0, 1], 128, b, out=out0.clone())
    for iy in range(3):
        for ix in range(2):
            tile = (0, slice(iy * 128, min(300, iy * 128 + 128)), slice(ix * 128, ix * 128 + 128))
            assert torch.equal(out[tile], out0[tile]) == (not info2[iy + 1, ix])


@pytest.mark.parametrize("p", [0.0, 0.5, 1.0])
def test_gemm_o_cache_plus_final_is_linear(p):
    g = torch.Generator().manual_seed(1)
    heads = 3
    x, w, b = torch.randn(2, 256, 384, generator=g), torch.randn(384, 384, generator=g), torch.randn(384, generator=g)
    info = np.random.default_rng(3).random((2, 2, heads)) < p
    segs = [np.packbits(info[i].reshape(-1).astype(np.uint8), bitorder="little") for i in range(2)]
    packed, indptr = np.concatenate(segs), [0, 1, 2]
    cache = oracle.gemm_o(x, w, heads, packed, indptr, 0, bias=b, is_for_cache=True)
    final = oracle.gemm_o(x, w, heads, packed, indptr, 0, bias=cache, is_for_cache=False)
    assert torch.allclose(final, F.linear(x, w, b), atol=1e-4)
    if p == 1.0:   # nothing cached: the cache pass is the broadcast bias
        assert torch.allclose(cache, b.expand_as(cache))
    if p == 0.0:   # everything cached: the cache pass is already the full layer
        assert torch.allclose(cache, F.linear(x, w, b), atol=1e-4)
    # per-mode closed form: masked-K matmul
    mask = torch.from_numpy(info).repeat_interleave(128, 1).repeat_interleave(128, 2)   # [B, M, K]
    assert torch.allclose(oracle.gemm_o(x, w, heads, packed, indptr, 0, is_for_cache=False),
                          (x * mask) @ w.T, atol=1e-4)


def test_quant_fp8_closed_forms():
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(300, 2, 128, generator=g) * 5).to(torch.bfloat16)
    x[128:256, 1] = 0
    x8, scale = oracle.quant_fp8_block(x, [0, 300])
    assert scale.shape == (2, 3) and float(scale[1, 1]) == 1.0
    for j, (a, b) in enumerate(((0, 128), (128, 256), (256, 300))):
        for h in range(2):
            amax = float(x[a:b, h].float().abs().max())
            if amax > 0:
                assert float(scale[h, j]) == pytest.approx(amax / 448.0, rel=1e-7)
                assert float(x8[a:b, h].float().abs().max()) == 448.0
                # same bytes as torch's own cast of the scaled block
                ref = (x[a:b, h].float() / scale[h, j]).to(torch.float8_e4m3fn)
                assert torch.equal(ref.view(torch.uint8), x8[a:b, h].view(torch.uint8))
    deq = oracle.dequant_fp8_block(x8, scale, [0, 300])
    err = (deq - x.float()).abs()
    assert bool((err <= x.float().abs() * 2 ** -4 + float(scale.max()) * 2 ** -9).all())


def test_fp8_attention_oracle_applies_scales():
    heads = 2
    q, k, v = _qkv(256, 384, heads, 7)
    m = make_ragged_masks([256], [384], heads, 1.0, 0.7, seed=1)
    q8, qs = oracle.quant_fp8_block(q, [0, 256])
    k8, ks = oracle.quant_fp8_block(k, [0, 384])
    a = oracle.sparse_attention(q8, k8, v, m["packed_info"], m["packed_keep"], m["info_indptr"], m["keep_indptr"],
                                m["qo_indptr"], m["kv_indptr"], q_scale=qs, k_scale=ks)
    qd = oracle.dequant_fp8_block(q8, qs, [0, 256])
    kd = oracle.dequant_fp8_block(k8, ks, [0, 384])
    b = oracle.sparse_attention(qd, kd, v.float(), m["packed_info"], m["packed_keep"], m["info_indptr"],
                                m["keep_indptr"], m["qo_indptr"], m["kv_indptr"])
    assert torch.allclose(a.float(), b, atol=2e-2)
    # against the unquantised inputs the error is the e4m3 rounding of q and k themselves: with 3
    # mantissa bits each element carries ~2.6% rms relative error, which for N(0,1) data becomes a
    # logit noise of ~0.037 and a relative L2 output error of about the same size
    ref = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"], m["keep_indptr"],
                                  m["qo_indptr"], m["kv_indptr"])
    assert 1e-2 < float((a.float() - ref.float()).norm() / ref.float().norm()) < 6e-2


@pytest.mark.parametrize("heads", [(4, 2), (6, 1), (14, 2)])
def test_attention_packed_tile_gqa_token_by_token(heads):
    """Grouped-query attention in the reference's symbol layout (prefill.cuh:410-413, 1283-1290),
    pinned by a second formulation that never forms a tile: for every (token, q head) on its own, the
    packed row is token * group + head % group, its tile row // 128, its kv head head // group; the
    symbol bit is tile * H_kv + kv_head and the kv bits follow at that index times the number of kv
    blocks; the output is the float64 softmax over the kept keys (masked SDPA).  A wrong divmod order,
    head base or bit index in the oracle moves rows between symbols and fails here."""
    hq, hkv = heads
    group = hq // hkv
    ql, kl = [150, 1, 260], [77, 300, 129]
    m = make_ragged_masks([n * group for n in ql], kl, hkv, 0.6, 0.5, seed=47)
    qo = np.concatenate([[0], np.cumsum(ql)]).astype(np.int32)
    kv = m["kv_indptr"]
    g = torch.Generator().manual_seed(47)
    q = torch.randn(sum(ql), hq, 128, generator=g)
    k = torch.randn(sum(kl), hkv, 128, generator=g)
    v = torch.randn(sum(kl), hkv, 128, generator=g)
    out0 = sentinel_like((sum(ql), hq, 128), torch.float32)
    lse = torch.full((sum(ql), hq), float("nan"))
    out = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"], m["keep_indptr"],
                                  qo, kv, out=out0.clone(), lse=lse, gqa_symbols="packed_tile")
    bit = lambda buf, base, i: (int(buf[base + i // 8]) >> (i % 8)) & 1
    c = math.log2(math.e) / math.sqrt(128)
    for r in range(len(ql)):
        nkv = -(-kl[r] // 128)
        for tok in range(ql[r]):
            for h in range(hq):
                row = tok * group + h % group
                sym = (row // 128) * hkv + h // group
                got = out[qo[r] + tok, h]
                if not bit(m["packed_info"], int(m["info_indptr"][r]), sym):
                    assert torch.equal(got, out0[qo[r] + tok, h]) and math.isnan(float(lse[qo[r] + tok, h]))
                    continue
                keys = [j for b in range(nkv) if bit(m["packed_keep"], int(m["keep_indptr"][r]), sym * nkv + b)
                        for j in range(kv[r] + b * 128, min(kv[r + 1], kv[r] + (b + 1) * 128))]
                if not keys:
                    assert float(got.abs().max()) == 0.0 and float(lse[qo[r] + tok, h]) == -5e4
                    continue
                s = (k[keys, h // group].double() @ q[qo[r] + tok, h].double()) * c
                p = torch.exp2(s - s.max())
                want = (p[:, None] * v[keys, h // group].double()).sum(0) / p.sum()
                assert float((got.double() - want).abs().max()) < 1e-4
                assert abs(float(lse[qo[r] + tok, h]) - float(torch.log2(p.sum()) + s.max())) < 1e-3


def test_attention_logits_soft_cap_token_by_token():
    """logits_soft_cap (variants.cuh:43-56, :68-70: logits -> tanh(q.k * sm_scale / cap), softmax scale
    log2(e) * cap) against a double-precision restatement written token by token with math.tanh, on
    logits large enough for the cap to bite; the base-2 lse with it.  Limits that a dropped factor would
    break: a huge cap is no cap; a tiny cap is the plain mean of the kept values (all scores within
    +-cap of each other, where a forgotten `* cap` would leave them within +-1)."""
    heads, n = 1, 128
    g = torch.Generator().manual_seed(9)
    q = torch.randn(n, heads, 128, generator=g) * 3
    k = torch.randn(2 * n, heads, 128, generator=g) * 3
    v = torch.randn(2 * n, heads, 128, generator=g)
    info = np.array([1], dtype=np.uint8)
    keep = np.packbits(np.array([0, 1], dtype=np.uint8), bitorder="little")   # second kv block only
    args = (info, keep, [0, 1], [0, 1], [0, n], [0, 2 * n])
    sm = 1.0 / math.sqrt(128)
    cap = 5.0
    lse = torch.zeros(n, heads)
    out = oracle.sparse_attention(q, k, v, *args, logits_soft_cap=cap, lse=lse)
    raw = (q[:, 0].double() @ k[n:, 0].double().T) * sm
    assert float(raw.abs().max()) > 2 * cap          # the cap matters on these logits
    for i in (0, 17, 127):
        sc = [cap * math.tanh(float(raw[i, j]) / cap) for j in range(n)]
        mx = max(sc)
        w = [math.exp(x - mx) for x in sc]
        tot = sum(w)
        ref = sum(w[j] * v[n + j, 0].double() for j in range(n)) / tot
        assert torch.allclose(out[i, 0].double(), ref, atol=1e-5, rtol=1e-4)
        assert abs(float(lse[i, 0]) - (math.log(tot) + mx) / math.log(2)) < 1e-4
    plain = oracle.sparse_attention(q, k, v, *args)
    assert not torch.allclose(out, plain, atol=1e-2)
    assert torch.allclose(oracle.sparse_attention(q, k, v, *args, logits_soft_cap=1e6), plain, atol=1e-4, rtol=1e-3)
    tiny = oracle.sparse_attention(q, k, v, *args, logits_soft_cap=1e-3)
    assert torch.allclose(tiny[:, 0], v[n:, 0].mean(0).expand(n, -1), atol=5e-3)
