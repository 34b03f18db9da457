"""GPU parity: sparse FlashAttention through the wrapper vs the fp32 dense masked oracle.

Tolerances are those stated for the path: bf16/fp16 outputs within max-abs 2e-2 and relative L2
1e-2 of the fp32 reference; skipped q-blocks byte-identical; listed rows without kv blocks zero."""
import math

import numpy as np
import pytest
import torch

import oracle
from helpers import make_ragged_masks, max_abs, rel_l2, sentinel_like

pytestmark = pytest.mark.gpu

MAX_ABS, REL_L2 = 2e-2, 1e-2


@pytest.fixture(autouse=True, params=["auto", "one_group"])
def kernel_variant(request):
    """Every test of this module runs twice: with the kernel form chosen from the list's size (short
    lists: one 8-wavefront workgroup per CU shares a row) and with the form for long lists forced
    (two 4-wavefront workgroups per CU, software-pipelined loop), which these small cases would not
    reach on their own.  Inputs the second form does not take (fp8) run the first one either way."""
    from flashomni_amd import _lib
    _lib.check(_lib.lib().fo_sparse_fa_set_variant(1 if request.param == "one_group" else 0))
    yield request.param
    _lib.check(_lib.lib().fo_sparse_fa_set_variant(0))


def _run_case(dev, ql, kl, heads, dtype, seed, pa=0.75, pk=0.5, force=None, is_full=False,
              return_lse=False, layout="NHD"):
    import flashomni_amd as fo
    m = make_ragged_masks(ql, kl, heads, pa, pk, seed=seed, force=force)
    g = torch.Generator().manual_seed(seed)
    nq, nk = int(m["qo_indptr"][-1]), int(m["kv_indptr"][-1])
    q = torch.randn(nq, heads, 128, generator=g).to(dtype)
    k = torch.randn(nk, heads, 128, generator=g).to(dtype)
    v = torch.randn(nk, heads, 128, generator=g).to(dtype)
    out0 = sentinel_like((nq, heads, 128), dtype)
    t = lambda a: torch.from_numpy(a).to(dev)
    ws = torch.empty(128 << 20, dtype=torch.uint8, device=dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(ws, layout)
    w.plan(t(m["qo_indptr"]), t(m["kv_indptr"]), heads, heads, 128, q_data_type=dtype)
    kd, vd = k.to(dev), v.to(dev)
    if layout == "HND":
        kd, vd = kd.transpose(0, 1).contiguous(), vd.transpose(0, 1).contiguous()
    out = out0.clone().to(dev)
    res = w.run(q.to(dev), kd, vd, t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]),
                t(m["keep_indptr"]), is_full, out=out, return_lse=return_lse)
    lse = None
    if return_lse:
        res, lse = res
    assert res.data_ptr() == out.data_ptr()
    exp_lse = torch.full((nq, heads), float("nan")) if return_lse else None
    exp = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"],
                                  m["keep_indptr"], m["qo_indptr"], m["kv_indptr"], is_full=is_full,
                                  out=out0.clone(), lse=exp_lse)
    return out.cpu(), exp, out0, m, (lse.cpu() if lse is not None else None), exp_lse


def _touched(m, heads, shape, is_full=False):
    """[token, head] mask of the rows that belong to listed (request, q-block, head) entries."""
    touched = torch.zeros(shape[:2], dtype=torch.bool)
    for r, info in enumerate(m["info"]):
        q0 = int(m["qo_indptr"][r])
        q1 = int(m["qo_indptr"][r + 1])
        for qb in range(info.shape[0]):
            for h in range(heads):
                if is_full or info[qb, h]:
                    touched[q0 + qb * 128:min(q1, q0 + (qb + 1) * 128), h] = True
    return touched


def _check(out, exp, out0, m, heads, is_full=False):
    # untouched q-blocks: byte-identical to the sentinel
    touched = _touched(m, heads, out.shape, is_full)
    assert torch.equal(out[~touched].view(torch.int16), out0[~touched].view(torch.int16))
    assert torch.equal(exp[~touched].view(torch.int16), out0[~touched].view(torch.int16))
    if touched.any():
        assert max_abs(out[touched], exp[touched]) <= MAX_ABS
        assert rel_l2(out[touched], exp[touched]) <= REL_L2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_small_single_request(dev, dtype):
    out, exp, out0, m, _, _ = _run_case(dev, [512], [512], 2, dtype, seed=1)
    _check(out, exp, out0, m, 2)


@pytest.mark.parametrize("layout", ["NHD", "HND"])
def test_ragged_batch_with_tails(dev, layout):
    ql, kl = [300, 1, 128, 1000, 129], [77, 513, 128, 1100, 64]
    out, exp, out0, m, _, _ = _run_case(dev, ql, kl, 3, torch.bfloat16, seed=2, layout=layout)
    _check(out, exp, out0, m, 3)


def test_requests_without_queries_or_without_keys(dev):
    """A batch holding a request with no q rows (nothing to do) and one with no keys (its active rows
    are rows without kv blocks: zeros, lse = -5e4, as prefill.cuh:385-386, :944-946 leave them), beside
    ordinary ones and a one-token request."""
    ql, kl = [200, 0, 128, 1], [300, 64, 0, 5]
    out, exp, out0, m, lse, exp_lse = _run_case(dev, ql, kl, 3, torch.bfloat16, seed=8, pa=0.8, pk=0.6,
                                                return_lse=True)
    _check(out, exp, out0, m, 3)
    ok = ~torch.isnan(exp_lse)
    assert ok.any() and float((lse[ok] - exp_lse[ok]).abs().max()) < 2e-2
    no_keys = slice(200, 328)   # the third request's rows
    act = torch.from_numpy(m["info"][2][0])           # its one q block, per head
    assert act.any()
    assert float(out[no_keys][:, act].abs().max()) == 0.0
    assert bool((lse[no_keys][:, act] == -5e4).all())


def test_all_ones_matches_sdpa(dev):
    """is_full and an all-ones mask both reduce to plain dense attention (a library routine)."""
    heads = 2
    for kwargs in (dict(force="ones"), dict(is_full=True)):
        out, exp, out0, m, _, _ = _run_case(dev, [384], [640], heads, torch.bfloat16, seed=3, **kwargs)
        _check(out, exp, out0, m, heads, is_full=True)


def test_all_cached_leaves_output_untouched(dev):
    out, exp, out0, m, _, _ = _run_case(dev, [384], [384], 2, torch.bfloat16, seed=4, force="zeros")
    assert torch.equal(out.view(torch.int16), out0.view(torch.int16))


def test_active_row_without_kv_blocks_writes_zeros_and_lse(dev):
    out, exp, out0, m, lse, exp_lse = _run_case(dev, [256], [256], 2, torch.bfloat16, seed=5, pa=1.0,
                                                pk=0.0, return_lse=True)
    assert float(out.abs().max()) == 0.0
    assert torch.equal(lse, torch.full_like(lse, -5e4))


def test_lse_base2(dev):
    out, exp, out0, m, lse, exp_lse = _run_case(dev, [300, 200], [500, 130], 2, torch.bfloat16, seed=6,
                                                pa=0.8, pk=0.6, return_lse=True)
    _check(out, exp, out0, m, 2)
    ok = ~torch.isnan(exp_lse)
    assert ok.any()
    assert float((lse[ok] - exp_lse[ok]).abs().max()) < 2e-2


def test_default_out_is_zero_filled(dev):
    import flashomni_amd as fo
    heads = 2
    m = make_ragged_masks([256], [256], heads, 0.5, 0.5, seed=11)
    t = lambda a: torch.from_numpy(a).to(dev)
    q = torch.randn(256, heads, 128, device=dev, dtype=torch.bfloat16)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w.plan(t(m["qo_indptr"]), t(m["kv_indptr"]), heads, heads, 128, q_data_type=torch.bfloat16)
    out = w.run(q, q, q, t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]))
    for qb in range(2):
        for h in range(heads):
            if not m["info"][0][qb, h]:
                assert float(out[qb * 128:(qb + 1) * 128, h].abs().max()) == 0.0


def test_flux_shape_full_config(dev):
    """Config 0 at full size (H=24, seq 4608): every active row checked against the oracle."""
    import flashomni_amd as fo
    from flashomni_amd.workloads import make_workload, sm_scale
    wl = make_workload(0)
    q, k, v = wl.tensors["q"], wl.tensors["k"], wl.tensors["v"]
    out0 = sentinel_like(q.shape, torch.bfloat16)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w.plan(wl.qo_indptr, wl.kv_indptr, 24, 24, 128, q_data_type=torch.bfloat16)
    out = out0.clone().to(dev)
    w.run(q.to(dev), k.to(dev), v.to(dev), wl.packed_info.to(dev), wl.packed_kv_info.to(dev),
          wl.info_indptr.to(dev), wl.kv_info_indptr.to(dev), out=out)
    exp = oracle.sparse_attention(q, k, v, wl.packed_info, wl.packed_kv_info, wl.info_indptr,
                                  wl.kv_info_indptr, wl.qo_indptr, wl.kv_indptr, out=out0.clone())
    out = out.cpu()
    active = wl.sparse_info.repeat_interleave(128, dim=0)[:4608]       # [seq, H]
    assert torch.equal(out[~active].view(torch.int16), out0[~active].view(torch.int16))
    assert max_abs(out[active], exp[active]) <= MAX_ABS
    assert rel_l2(out[active], exp[active]) <= REL_L2


def test_dtype_mismatch_and_missing_symbols_raise(dev):
    import flashomni_amd as fo
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    ip = torch.tensor([0, 128], dtype=torch.int32, device=dev)
    w.plan(ip, ip, 1, 1, 128, q_data_type=torch.bfloat16)
    q = torch.zeros(128, 1, 128, device=dev, dtype=torch.float16)
    with pytest.raises(ValueError, match="does not match the q_data_type"):
        w.run(q, q, q, is_full=True)
    q = q.to(torch.bfloat16)
    with pytest.raises(ValueError, match="required unless"):
        w.run(q, q, q)
    with pytest.raises(ValueError, match="Invalid shape of out"):
        w.run(q, q, q, is_full=True, out=torch.zeros(64, 1, 128, device=dev, dtype=torch.bfloat16))


def test_undersized_tensors_raise(dev):
    """Tensors smaller than the planned batch are refused on the host: the kernels index by the
    planned token counts and symbol layout."""
    import flashomni_amd as fo
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    qo = torch.tensor([0, 300, 556], dtype=torch.int32, device=dev)      # 3 + 2 q blocks
    kv = torch.tensor([0, 256, 700], dtype=torch.int32, device=dev)      # 2 + 4 kv blocks
    w.plan(qo, kv, 4, 4, 128, q_data_type=torch.bfloat16)
    q = torch.zeros(556, 4, 128, device=dev, dtype=torch.bfloat16)
    k = torch.zeros(700, 4, 128, device=dev, dtype=torch.bfloat16)
    info = torch.zeros(2 + 1, dtype=torch.uint8, device=dev)             # ceil(12/8) + ceil(8/8)
    keep = torch.zeros(3 + 4, dtype=torch.uint8, device=dev)             # ceil(24/8) + ceil(32/8)
    ip = torch.tensor([0, 2, 3], dtype=torch.int32, device=dev)
    kp = torch.tensor([0, 3, 7], dtype=torch.int32, device=dev)
    w.run(q, k, k, info, keep, ip, kp)
    with pytest.raises(ValueError, match="tokens; the planned"):
        w.run(q[:500], k, k, info, keep, ip, kp)
    with pytest.raises(ValueError, match="tokens; the planned"):
        w.run(q, k[:600], k[:600], info, keep, ip, kp)
    with pytest.raises(ValueError, match="sparse_info holds 2 bytes"):
        w.run(q, k, k, info[:2], keep, ip, kp)
    with pytest.raises(ValueError, match="sparse_kv_info holds 6 bytes"):
        w.run(q, k, k, info, keep[:6], ip, kp)
    with pytest.raises(ValueError, match="must have 3 entries"):
        w.run(q, k, k, info, keep, ip[:2], kp)
    with pytest.raises(ValueError, match="3-dimensional"):
        w.run(q[:, 0], k, k, info, keep, ip, kp)


# ------------------------------------------------------------------------------------------------
# fp8 (e4m3fn) Q.K^T path.  The reference has no fp8 matrix product (it up-casts fp8 storage to
# fp16) and no absmax quantiser: parity unpinned against it.  Two checks:
#  * kernel parity: against the fp32 dense masked oracle fed with the SAME quantised q/k bytes and
#    scales -> relative L2 <= 3e-2 (the stated fp8 tolerance), max-abs <= 2e-2;
#  * end to end against the unquantised fp32 reference: e4m3 keeps 3 mantissa bits, i.e. ~2.6% rms
#    relative error per element of q and k, which for N(0,1) data is a logit noise of ~0.037 and a
#    relative L2 output error of the same size -- above 3e-2 whatever the kernel does.  The test
#    pins the measured error to that analytic level (< 6e-2).
# ------------------------------------------------------------------------------------------------
FP8_REL_L2 = 3e-2


@pytest.mark.parametrize("two_term", [True, False, "qk"])
@pytest.mark.parametrize("case", [([512], [512], 2), ([300, 1, 128, 1000, 129], [77, 513, 128, 1100, 64], 3)])
def test_fp8_attention(dev, case, two_term):
    """fp8 q and k with per-(head, block) scales.  Against the oracle fed the same quantised operands the
    kernel has to be as exact as the 16-bit one.  Against the unquantised fp32 oracle the stated 3e-2
    holds for the two-term q (q + q_lo: only k's rounding is left in the logits); a one-term q is a
    faster form outside that contract (two e4m3 roundings per product: ~3.9e-2 on unit-variance data).
    "qk": k in two terms as well (k + k_lo): the logits are then as accurate as 16-bit ones."""
    import flashomni_amd as fo
    ql, kl, heads = case
    m = make_ragged_masks(ql, kl, heads, 0.75, 0.5, seed=21)
    g = torch.Generator().manual_seed(21)
    nq, nk = int(m["qo_indptr"][-1]), int(m["kv_indptr"][-1])
    q = torch.randn(nq, heads, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(nk, heads, 128, generator=g).to(torch.bfloat16)
    v = torch.randn(nk, heads, 128, generator=g).to(torch.bfloat16)
    t = lambda a: torch.from_numpy(a).to(dev)
    q8, qs, q_lo = fo.quant_fp8_block(q.to(dev), torch.from_numpy(m["qo_indptr"]), residual=True)
    if not two_term:
        q_lo = None
    k8, ks, k_lo = fo.quant_fp8_block(k.to(dev), torch.from_numpy(m["kv_indptr"]), residual=True)
    if two_term != "qk":
        k_lo = None
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w.plan(t(m["qo_indptr"]), t(m["kv_indptr"]), heads, heads, 128, q_data_type=torch.float8_e4m3fn)
    out0 = sentinel_like((nq, heads, 128), torch.bfloat16)
    out = out0.clone().to(dev)
    lse = torch.full((nq, heads), float("nan"), device=dev)
    w.run(q8, k8, v.to(dev), t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]),
          t(m["keep_indptr"]), out=out, lse=lse, return_lse=True, q_scale=qs, k_scale=ks, q_lo=q_lo, k_lo=k_lo)
    exp_lse = torch.full((nq, heads), float("nan"))
    exp = oracle.sparse_attention(q8.cpu(), k8.cpu(), v, m["packed_info"], m["packed_keep"], m["info_indptr"],
                                  m["keep_indptr"], m["qo_indptr"], m["kv_indptr"], out=out0.clone(),
                                  lse=exp_lse, q_scale=qs.cpu(), k_scale=ks.cpu(),
                                  q_lo=None if q_lo is None else q_lo.cpu(),
                                  k_lo=None if k_lo is None else k_lo.cpu())
    out = out.cpu()
    changed = _touched(m, heads, out.shape)
    assert torch.equal(out[~changed].view(torch.int16), out0[~changed].view(torch.int16))
    assert rel_l2(out[changed], exp[changed]) <= REL_L2
    assert max_abs(out[changed], exp[changed]) <= MAX_ABS
    ok = ~torch.isnan(exp_lse)
    assert float((lse.cpu()[ok] - exp_lse[ok]).abs().max()) < 2e-2
    ref = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"],
                                  m["keep_indptr"], m["qo_indptr"], m["kv_indptr"], out=out0.clone())
    err = rel_l2(out[changed], ref[changed])
    print("fp8 attention vs the unquantised oracle, terms %s: rel-L2 %.4g" % (two_term, err))
    if two_term == "qk":
        assert err <= REL_L2       # two terms on both sides: the 16-bit tolerance
    elif two_term:
        assert err <= FP8_REL_L2   # the stated fp8 tolerance
    else:
        assert err <= 4.5e-2       # not the contract: the level two e4m3 operands explain


@pytest.mark.parametrize("config", [4])
def test_fp8_attention_video_shape_sampled_rows(dev, config):
    """fp8 attention (two-term q) at config 4's full size on unit-variance q, k, v: sampled rows within the
    stated relative L2 3e-2 of the unquantised fp32 oracle."""
    import flashomni_amd as fo
    from flashomni_amd.workloads import make_workload
    wl = make_workload(config, tensors=False)
    s = wl.shape
    g = torch.Generator(device=dev).manual_seed(300 + config)
    draw = lambda: torch.randn(s.seq, s.heads, 128, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    q, k, v = draw(), draw(), draw()
    q8, qs, q_lo = fo.quant_fp8_block(q, wl.qo_indptr, residual=True)
    k8, ks = fo.quant_fp8_block(k, wl.kv_indptr)
    out = torch.full((s.seq, s.heads, 128), -7.0, dtype=torch.bfloat16, device=dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(256 << 20, dtype=torch.uint8, device=dev))
    w.plan(wl.qo_indptr, wl.kv_indptr, s.heads, s.heads, 128, q_data_type=torch.float8_e4m3fn)
    w.run(q8, k8, v, wl.packed_info.to(dev), wl.packed_kv_info.to(dev), wl.info_indptr.to(dev),
          wl.kv_info_indptr.to(dev), out=out, q_scale=qs, k_scale=ks, q_lo=q_lo)
    torch.cuda.synchronize()
    active = wl.sparse_info.to(dev).repeat_interleave(128, dim=0)[:s.seq]
    assert bool((out[~active] == -7.0).all())
    _, row_qb, row_head, ptr, _ = oracle.decode_kv_csr(
        wl.packed_info.numpy(), wl.packed_kv_info.numpy(), wl.info_indptr.numpy(),
        wl.kv_info_indptr.numpy(), wl.qo_indptr.numpy(), wl.kv_indptr.numpy(), s.heads, 128, 128)
    edge = np.nonzero((row_qb == 0) | (row_qb == s.n_blocks - 1))[0]
    rng = np.random.default_rng(config)
    rows = np.unique(np.concatenate([edge, rng.choice(len(row_qb), 64, replace=False)]))
    exp = torch.full((s.seq, s.heads, 128), -7.0, dtype=torch.bfloat16)
    oracle.sparse_attention(q.cpu(), k.cpu(), v.cpu(), wl.packed_info, wl.packed_kv_info,
                            wl.info_indptr, wl.kv_info_indptr, wl.qo_indptr, wl.kv_indptr,
                            out=exp, rows=[int(i) for i in rows])
    got = out.cpu()
    num, den = 0.0, 0.0
    for i in rows:
        q0 = int(row_qb[i]) * 128
        sl = (slice(q0, min(s.seq, q0 + 128)), int(row_head[i]))
        a, b = got[sl].float(), exp[sl].float()
        num += float(((a - b) ** 2).sum())
        den += float((b ** 2).sum())
    print("fp8 attention at config %d, two-term q: rel-L2 %.4g" % (config, math.sqrt(num / den)))
    assert math.sqrt(num / den) <= FP8_REL_L2


def test_fp8_attention_needs_scales(dev):
    import flashomni_amd as fo
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    ip = torch.tensor([0, 128], dtype=torch.int32, device=dev)
    w.plan(ip, ip, 1, 1, 128, q_data_type=torch.float8_e4m3fn)
    q8 = torch.zeros(128, 1, 128, device=dev, dtype=torch.float8_e4m3fn)
    v = torch.zeros(128, 1, 128, device=dev, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="q_scale and k_scale"):
        w.run(q8, q8, v, is_full=True)


@pytest.mark.parametrize("sign", [1.0, -1.0])
def test_logits_that_move_the_running_max(dev, sign):
    """Keys whose logits grow along the sequence (the running reference point has to be raised many
    times), and the mirrored case where every logit is far below zero (the first tile has to
    re-centre downwards): both against the fp32 oracle, output and base-2 lse."""
    import flashomni_amd as fo
    heads, nq, nk = 2, 256, 2048 + 37
    m = make_ragged_masks([nq], [nk], heads, 1.0, 0.7, seed=21)
    g = torch.Generator().manual_seed(21)
    q = torch.randn(nq, heads, 128, generator=g)
    k = torch.randn(nk, heads, 128, generator=g) * 0.3
    # a component along q's mean direction that grows with the key position: the logits drift by
    # about 24 in the log2 domain over the sequence
    drift = torch.linspace(1.0, 2.0, nk).view(nk, 1, 1) * sign
    k = k + drift * torch.ones(1, heads, 128) * 1.5
    q = q + 1.0
    v = torch.randn(nk, heads, 128, generator=g)
    q, k, v = (x.to(torch.bfloat16) for x in (q, k, v))
    t = lambda a: torch.from_numpy(a).to(dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w.plan(t(m["qo_indptr"]), t(m["kv_indptr"]), heads, heads, 128, q_data_type=torch.bfloat16)
    out, lse = w.run(q.to(dev), k.to(dev), v.to(dev), t(m["packed_info"]), t(m["packed_keep"]),
                     t(m["info_indptr"]), t(m["keep_indptr"]), return_lse=True)
    exp_lse = torch.full((nq, heads), float("nan"))
    exp = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"],
                                  m["keep_indptr"], m["qo_indptr"], m["kv_indptr"],
                                  out=torch.zeros(nq, heads, 128, dtype=torch.bfloat16), lse=exp_lse)
    x = torch.einsum("qhd,khd->hqk", q.float(), k.float()) * (128 ** -0.5) * 1.4426950408889634
    assert float(x.max() - x.min()) > 16.0          # the case really leaves the lazy window of 2^8
    assert sign > 0 or float(x.max()) < -8.0        # mirrored case: every logit far below zero
    assert max_abs(out.cpu(), exp) <= MAX_ABS and rel_l2(out.cpu(), exp) <= REL_L2
    # |logits| reach ~50 here: the one extra bf16 rounding of q (scale folded into Q) shows as a
    # relative error of the lse
    assert float(((lse.cpu() - exp_lse).abs() / (1.0 + exp_lse.abs())).max()) < 2e-3


def _split_case(dev, ql, kl, heads, seed, share, dtype=torch.bfloat16, pk=0.6):
    """Run one launch (twice, to see the arrival counters re-armed) with or without rows shared
    between workgroups; returns (out, lse, sched words, expectations)."""
    import flashomni_amd as fo
    m = make_ragged_masks(ql, kl, heads, 1.0, pk, seed=seed)
    g = torch.Generator().manual_seed(seed)
    nq, nk = int(m["qo_indptr"][-1]), int(m["kv_indptr"][-1])
    q = torch.randn(nq, heads, 128, generator=g).to(dtype)
    k = torch.randn(nk, heads, 128, generator=g).to(dtype)
    v = torch.randn(nk, heads, 128, generator=g).to(dtype)
    t = lambda a: torch.from_numpy(a).to(dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(64 << 20, dtype=torch.uint8, device=dev))
    w._share_rows = share
    w.plan(t(m["qo_indptr"]), t(m["kv_indptr"]), heads, heads, 128, q_data_type=dtype)
    args = (t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]))
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    out1, lse1 = w.run(qd, kd, vd, *args, return_lse=True)
    out1, lse1 = out1.clone(), lse1.clone()
    out2, lse2 = w.run(qd, kd, vd, *args, return_lse=True)
    assert torch.equal(out1, out2) and torch.equal(lse1, lse2), "second launch over the same list differs"
    sched = w._worklist.sched.cpu().numpy()
    exp_lse = torch.full((nq, heads), float("nan"))
    exp = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"],
                                  m["keep_indptr"], m["qo_indptr"], m["kv_indptr"],
                                  out=torch.zeros(nq, heads, 128, dtype=dtype), lse=exp_lse)
    return out2.cpu(), lse2.cpu(), sched, exp, exp_lse


@pytest.mark.parametrize("case", [
    ([1024], [4096], 2),             # 16 rows of ~19 blocks: every row cut in up to four parts
    ([1536], [2048 + 77], 8),        # 96 rows, ragged kv tail in a last part
    ([128 * 9], [128 * 9], 1),       # 9 short rows in one head
    ([1536, 640], [2304, 1500], 24),   # 1.6 rows per CU: most workgroups end in a shared row
])
def test_rows_shared_between_workgroups(dev, case):
    """Few rows per CU: the decoder lays out even shares, rows that straddle a share boundary are
    computed in parts and combined by the last arrival.  Checked against the oracle, against the
    same launch with sharing switched off (every row computed whole from the queues), and for the
    counters being left re-armed."""
    ql, kl, heads = case
    out, lse, sched, exp, exp_lse = _split_case(dev, ql, kl, heads, seed=31, share=True)
    assert sched[26] == 1 and sched[27] > 0
    assert (sched[64:576] == 0).all() and (sched[16:25] == 0).all()
    assert max_abs(out, exp) <= MAX_ABS and rel_l2(out, exp) <= REL_L2
    assert torch.allclose(lse, exp_lse, atol=2e-3, rtol=1e-3)
    whole, lse_w, sched_w, _, _ = _split_case(dev, ql, kl, heads, seed=31, share=False)
    assert sched_w[26] == 0                     # the decoder was given no share table
    assert max_abs(out, whole) <= 8e-3          # same math, the parts' sums are combined in another order
    assert torch.allclose(lse, lse_w, atol=1e-3, rtol=1e-4)


def test_shared_rows_fp8(dev):
    import flashomni_amd as fo
    ql, kl, heads = [1024], [2048], 2
    m = make_ragged_masks(ql, kl, heads, 1.0, 0.7, seed=33)
    g = torch.Generator().manual_seed(33)
    q = torch.randn(ql[0], heads, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(kl[0], heads, 128, generator=g).to(torch.bfloat16)
    v = torch.randn(kl[0], heads, 128, generator=g).to(torch.bfloat16)
    t = lambda a: torch.from_numpy(a).to(dev)
    args = (t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]))
    outs = []
    for share in (True, False):
        w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(64 << 20, dtype=torch.uint8, device=dev))
        w._share_rows = share
        w.plan(t(m["qo_indptr"]), t(m["kv_indptr"]), heads, heads, 128, q_data_type=torch.float8_e4m3fn)
        q8, qs = fo.quant_fp8_block(q.to(dev), t(m["qo_indptr"]))
        k8, ks = fo.quant_fp8_block(k.to(dev), t(m["kv_indptr"]))
        outs.append(w.run(q8, k8, v.to(dev), *args, q_scale=qs, k_scale=ks).cpu())
        assert w._worklist.sched.cpu().numpy()[26] == int(share)
    assert max_abs(outs[0], outs[1]) <= 8e-3


@pytest.mark.parametrize("heads", [(4, 2), (6, 1), (8, 8)])
@pytest.mark.parametrize("layout", ["NHD", "HND"])
def test_grouped_query_attention(dev, heads, layout):
    """num_kv_heads < num_qo_heads: q head h reads kv head h / group (prefill.cuh:410-413)."""
    import flashomni_amd as fo
    hq, hkv = heads
    ql, kl = [300, 1, 640], [77, 513, 640]
    m = make_ragged_masks(ql, kl, hq, 0.8, 0.5, seed=41)
    g = torch.Generator().manual_seed(41)
    nq, nk = sum(ql), sum(kl)
    q = torch.randn(nq, hq, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(nk, hkv, 128, generator=g).to(torch.bfloat16)
    v = torch.randn(nk, hkv, 128, generator=g).to(torch.bfloat16)
    t = lambda a: torch.from_numpy(a).to(dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(256 << 20, dtype=torch.uint8, device=dev), layout)
    w.plan(t(m["qo_indptr"]), t(m["kv_indptr"]), hq, hkv, 128, q_data_type=torch.bfloat16,
           gqa_symbols="per_q_head")
    kd, vd = k.to(dev), v.to(dev)
    if layout == "HND":
        kd, vd = kd.transpose(0, 1).contiguous(), vd.transpose(0, 1).contiguous()
    out0 = sentinel_like((nq, hq, 128), torch.bfloat16)
    out, lse = w.run(q.to(dev), kd, vd, t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]),
                     t(m["keep_indptr"]), out=out0.clone().to(dev), return_lse=True)
    exp_lse = torch.full((nq, hq), float("nan"))
    exp = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"],
                                  m["keep_indptr"], m["qo_indptr"], m["kv_indptr"], out=out0.clone(), lse=exp_lse)
    _check(out.cpu(), exp, out0, m, hq)
    ok = ~torch.isnan(exp_lse)
    assert torch.allclose(lse.cpu()[ok], exp_lse[ok], atol=2e-3, rtol=1e-3)
    with pytest.raises(ValueError, match="kv head count"):
        w.run(q.to(dev), torch.zeros(nk, hkv + 1, 128, dtype=torch.bfloat16, device=dev).transpose(0, 1 if layout == "HND" else 0),
              vd, t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]))
    with pytest.raises(ValueError, match="multiple of num_kv_heads"):
        w.plan(t(m["qo_indptr"]), t(m["kv_indptr"]), 6, 4, 128, q_data_type=torch.bfloat16)


@pytest.mark.parametrize("heads", [(4, 2), (6, 1), (8, 2), (14, 2)])
@pytest.mark.parametrize("layout", ["NHD", "HND"])
def test_grouped_query_attention_packed_tiles(dev, heads, layout):
    """The reference's symbol layout for num_kv_heads < num_qo_heads (prefill.cuh:410-413, 1283-1290):
    one symbol per (tile of 128 packed (token, q head) rows, kv head).  Groups of 2, 4, 6 and 7 q heads:
    with 6 and 7 a tile ends in the middle of a token's heads.  Rows of tiles that are not listed keep
    their bytes (which rows those are is worked out here from the flags, token by token)."""
    import flashomni_amd as fo
    hq, hkv = heads
    group = hq // hkv
    ql, kl = [300, 1, 640], [77, 513, 640]
    # symbols of the packed layout: a request of qo_len tokens has ceil(qo_len * group / 128) tiles
    m = make_ragged_masks([n * group for n in ql], kl, hkv, 0.7, 0.5, seed=43)
    qo_indptr = np.concatenate([[0], np.cumsum(ql)]).astype(np.int32)
    g = torch.Generator().manual_seed(43)
    nq, nk = sum(ql), sum(kl)
    q = torch.randn(nq, hq, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(nk, hkv, 128, generator=g).to(torch.bfloat16)
    v = torch.randn(nk, hkv, 128, generator=g).to(torch.bfloat16)
    t = lambda a: torch.from_numpy(a).to(dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(256 << 20, dtype=torch.uint8, device=dev), layout)
    w.plan(t(qo_indptr), t(m["kv_indptr"]), hq, hkv, 128, q_data_type=torch.bfloat16)  # the default layout
    kd, vd = k.to(dev), v.to(dev)
    if layout == "HND":
        kd, vd = kd.transpose(0, 1).contiguous(), vd.transpose(0, 1).contiguous()
    out0 = sentinel_like((nq, hq, 128), torch.bfloat16)
    out, lse = w.run(q.to(dev), kd, vd, t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]),
                     t(m["keep_indptr"]), out=out0.clone().to(dev), return_lse=True)
    exp_lse = torch.full((nq, hq), float("nan"))
    exp = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"],
                                  m["keep_indptr"], qo_indptr, m["kv_indptr"], out=out0.clone(), lse=exp_lse,
                                  gqa_symbols="packed_tile")
    touched = torch.zeros(nq, hq, dtype=torch.bool)
    for r, n in enumerate(ql):
        for tok in range(n):
            for h in range(hq):
                tile = (tok * group + h % group) // 128
                touched[qo_indptr[r] + tok, h] = bool(m["info"][r][tile, h // group])
    out = out.cpu()
    assert torch.equal(out[~touched].view(torch.int16), out0[~touched].view(torch.int16))
    assert touched.any() and not touched.all()
    assert max_abs(out[touched], exp[touched]) <= MAX_ABS
    assert rel_l2(out[touched], exp[touched]) <= REL_L2
    assert torch.equal(~torch.isnan(exp_lse), touched)
    # (absolute: the kernel sums probabilities that were rounded to bf16 for the P.V product, so the
    # base-2 logarithm of a sum of few terms is off by a few 2^-9 / ln 2 = 2.8e-3 whatever its size; the
    # one-token request here has such rows with lse near 0, where a relative bound allows nothing)
    assert float((lse.cpu()[touched] - exp_lse[touched]).abs().max()) <= 8e-3
    # fp8 q carries one scale per (q head, token block): not available for tiles of several q heads
    w.plan(t(qo_indptr), t(m["kv_indptr"]), hq, hkv, 128, q_data_type=torch.float8_e4m3fn)
    q8, qs = fo.quant_fp8_block(q.to(dev), t(qo_indptr))
    k8, ks = fo.quant_fp8_block(k.to(dev), t(m["kv_indptr"]))
    with pytest.raises(NotImplementedError, match="packed tiles"):
        w.run(q8, k8 if layout == "NHD" else k8.transpose(0, 1).contiguous(), vd, t(m["packed_info"]),
              t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]), q_scale=qs, k_scale=ks)


@pytest.mark.parametrize("config", [3, 4])
def test_video_shapes_sampled_rows(dev, config):
    """Configs 3 and 4 at full size (H=24, seq 33 280 and H=40, seq 76 112 with a ragged last block): the kernel runs
    the whole work list; every row of the first and last q-block plus 64 seeded random rows are
    checked against the oracle, and skipped (q-block, head) strips keep their bytes."""
    import flashomni_amd as fo
    from flashomni_amd.workloads import make_workload
    wl = make_workload(config, tensors=False)
    s = wl.shape
    g = torch.Generator(device=dev).manual_seed(100 + config)
    draw = lambda: torch.randn(s.seq, s.heads, 128, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    q, k, v = draw(), draw(), draw()
    out = torch.full((s.seq, s.heads, 128), -7.0, dtype=torch.bfloat16, device=dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(256 << 20, dtype=torch.uint8, device=dev))
    w.plan(wl.qo_indptr, wl.kv_indptr, s.heads, s.heads, 128, q_data_type=torch.bfloat16)
    w.run(q, k, v, wl.packed_info.to(dev), wl.packed_kv_info.to(dev), wl.info_indptr.to(dev),
          wl.kv_info_indptr.to(dev), out=out)
    torch.cuda.synchronize()

    active = wl.sparse_info.to(dev).repeat_interleave(128, dim=0)[:s.seq]      # [seq, H]
    assert bool((out[~active] == -7.0).all())
    assert bool(torch.isfinite(out[active].float()).all())

    _, row_qb, row_head, ptr, _ = oracle.decode_kv_csr(
        wl.packed_info.numpy(), wl.packed_kv_info.numpy(), wl.info_indptr.numpy(),
        wl.kv_info_indptr.numpy(), wl.qo_indptr.numpy(), wl.kv_indptr.numpy(), s.heads, 128, 128)
    edge = np.nonzero((row_qb == 0) | (row_qb == s.n_blocks - 1))[0]
    rng = np.random.default_rng(config)
    rows = np.unique(np.concatenate([edge, rng.choice(len(row_qb), 64, replace=False)]))
    assert (row_qb[rows] == s.n_blocks - 1).any()                              # the short block is covered
    exp = torch.full((s.seq, s.heads, 128), -7.0, dtype=torch.bfloat16)
    oracle.sparse_attention(q.cpu(), k.cpu(), v.cpu(), wl.packed_info, wl.packed_kv_info,
                            wl.info_indptr, wl.kv_info_indptr, wl.qo_indptr, wl.kv_indptr,
                            out=exp, rows=[int(i) for i in rows])
    got = out.cpu()
    worst_abs, num, den = 0.0, 0.0, 0.0
    for i in rows:
        q0 = int(row_qb[i]) * 128
        sl = (slice(q0, min(s.seq, q0 + 128)), int(row_head[i]))
        a, b = got[sl].float(), exp[sl].float()
        worst_abs = max(worst_abs, float((a - b).abs().max()))
        num += float(((a - b) ** 2).sum())
        den += float((b ** 2).sum())
    assert worst_abs <= MAX_ABS
    assert math.sqrt(num / den) <= REL_L2


def test_two_wrappers_on_two_streams(dev):
    """Two planned wrappers (own workspaces, own work lists) launched back to back on two streams
    without synchronising in between: the library keeps no state that the launches could share."""
    import flashomni_amd as fo
    cases = []
    for seed, (ql, kl, heads) in enumerate([([700, 260], [900, 300], 8), ([1536], [2048], 16)]):
        m = make_ragged_masks(ql, kl, heads, 0.7, 0.5, seed=50 + seed)
        g = torch.Generator().manual_seed(60 + seed)
        nq, nk = int(m["qo_indptr"][-1]), int(m["kv_indptr"][-1])
        q = torch.randn(nq, heads, 128, generator=g).to(torch.bfloat16)
        k = torch.randn(nk, heads, 128, generator=g).to(torch.bfloat16)
        v = torch.randn(nk, heads, 128, generator=g).to(torch.bfloat16)
        t = lambda a: torch.from_numpy(a).to(dev)
        w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(64 << 20, dtype=torch.uint8, device=dev))
        w.plan(t(m["qo_indptr"]), t(m["kv_indptr"]), heads, heads, 128, q_data_type=torch.bfloat16)
        dev_args = (q.to(dev), k.to(dev), v.to(dev), t(m["packed_info"]), t(m["packed_keep"]),
                    t(m["info_indptr"]), t(m["keep_indptr"]))
        out0 = sentinel_like((nq, heads, 128), torch.bfloat16)
        exp = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"],
                                      m["keep_indptr"], m["qo_indptr"], m["kv_indptr"], out=out0.clone())
        cases.append((w, dev_args, out0, exp, m, heads, torch.cuda.Stream(device=dev)))
    torch.cuda.synchronize()
    outs = []
    for rep in range(3):
        outs = []
        for w, dev_args, out0, exp, m, heads, stream in cases:
            with torch.cuda.stream(stream):
                out = out0.clone().to(dev, non_blocking=False)
                w.run(*dev_args, out=out)
                outs.append(out)
    torch.cuda.synchronize()
    for out, (w, dev_args, out0, exp, m, heads, stream) in zip(outs, cases):
        _check(out.cpu(), exp, out0, m, heads)


@pytest.mark.parametrize("seed", range(16))
def test_random_ragged_batches(dev, seed):
    """Seeded random batches (1-4 requests, ragged lengths down to one token, 1-12 heads, random
    densities, either dtype, either layout; short lists, so the rows are cut into even shares)
    against the oracle, lse included."""
    rng = np.random.default_rng(1000 + seed)
    n_req = int(rng.integers(1, 5))
    ql = [int(rng.integers(1, 900)) for _ in range(n_req)]
    kl = [int(rng.integers(1, 1400)) for _ in range(n_req)]
    heads = int(rng.choice([1, 2, 3, 5, 8, 12]))
    pa, pk = float(rng.choice([0.3, 0.7, 1.0])), float(rng.choice([0.1, 0.5, 0.9]))
    dtype = torch.bfloat16 if seed % 2 == 0 else torch.float16
    layout = "NHD" if seed % 3 else "HND"
    out, exp, out0, m, lse, exp_lse = _run_case(dev, ql, kl, heads, dtype, seed=2000 + seed, pa=pa, pk=pk,
                                                return_lse=True, layout=layout)
    _check(out, exp, out0, m, heads)
    ok = ~torch.isnan(exp_lse)
    assert torch.allclose(lse[ok], exp_lse[ok], atol=2e-3, rtol=1e-3)


def test_share_with_many_short_rows(dev):
    """One long row (150 kv blocks, cut into parts) beside 80 rows without any kv block: the
    long row sets the share size, so single shares hold more than sixteen of the short rows (their
    records are gathered in batches of sixteen)."""
    import flashomni_amd as fo
    heads, ql, kl = 1, [128, 80 * 128], [150 * 128, 128]
    info = [np.ones((1, 1), dtype=bool), np.ones((80, 1), dtype=bool)]
    keep = [np.ones((1, 1, 150), dtype=bool), np.zeros((80, 1, 1), dtype=bool)]
    pack = lambda parts: (np.concatenate([np.packbits(p.reshape(-1), bitorder="little") for p in parts]),
                          np.cumsum([0] + [(p.size + 7) // 8 for p in parts]).astype(np.int32))
    pinfo, info_ip = pack(info)
    pkeep, keep_ip = pack(keep)
    qo, kv = np.array([0, 128, 128 + 80 * 128], dtype=np.int32), np.array([0, 150 * 128, 151 * 128], dtype=np.int32)
    g = torch.Generator().manual_seed(9)
    q = torch.randn(int(qo[-1]), heads, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(int(kv[-1]), heads, 128, generator=g).to(torch.bfloat16)
    v = torch.randn(int(kv[-1]), heads, 128, generator=g).to(torch.bfloat16)
    t = lambda a: torch.from_numpy(a).to(dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w.plan(t(qo), t(kv), heads, heads, 128, q_data_type=torch.bfloat16)
    out0 = sentinel_like(q.shape, torch.bfloat16)
    out = out0.clone().to(dev)
    w.run(q.to(dev), k.to(dev), v.to(dev), t(pinfo), t(pkeep), t(info_ip), t(keep_ip), out=out)
    sched = w._worklist.sched.cpu().numpy()
    assert sched[26] == 1 and sched[27] == 50 and sched[30] == 81   # share = ceil((150 + 2) / 3)
    exp = oracle.sparse_attention(q, k, v, pinfo, pkeep, info_ip, keep_ip, qo, kv, out=out0.clone())
    out = out.cpu()
    assert float(out[128:].abs().max()) == 0.0 and float(exp[128:].abs().max()) == 0.0
    assert max_abs(out[:128], exp[:128]) <= MAX_ABS and rel_l2(out[:128], exp[:128]) <= REL_L2


@pytest.mark.parametrize("cap", [1.0, 30.0])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_logits_soft_cap(dev, cap, dtype):
    """plan(..., logits_soft_cap=cap) (reference: flashomni/attention.py:421-429 -> variants.cuh:43-56,
    :68-70): scores cap * tanh(q.k * sm_scale / cap), on a ragged batch with tails, q scaled so that the
    raw logits reach several times the smaller cap; output within the path's tolerances of the oracle,
    lse (base 2, over the capped scores) within 2e-2, skipped q blocks untouched.  The kernel form with
    the cap is the 8-wavefront one whatever the list's length, so both settings of the fixture run it."""
    import flashomni_amd as fo
    heads = 3
    ql, kl = [300, 1, 640], [77, 513, 700]
    m = make_ragged_masks(ql, kl, heads, 0.8, 0.6, seed=21)
    g = torch.Generator().manual_seed(21)
    nq, nk = sum(ql), sum(kl)
    q = (torch.randn(nq, heads, 128, generator=g) * 2).to(dtype)
    k = torch.randn(nk, heads, 128, generator=g).to(dtype)
    v = torch.randn(nk, heads, 128, generator=g).to(dtype)
    out0 = sentinel_like((nq, heads, 128), dtype)
    t = lambda a: torch.from_numpy(a).to(dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w.plan(t(m["qo_indptr"]), t(m["kv_indptr"]), heads, heads, 128, q_data_type=dtype, logits_soft_cap=cap)
    out = out0.clone().to(dev)
    _, lse = w.run(q.to(dev), k.to(dev), v.to(dev), t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]),
                   t(m["keep_indptr"]), out=out, return_lse=True)
    exp_lse = torch.full((nq, heads), float("nan"))
    sym = (m["packed_info"], m["packed_keep"], m["info_indptr"], m["keep_indptr"], m["qo_indptr"], m["kv_indptr"])
    exp = oracle.sparse_attention(q, k, v, *sym, out=out0.clone(), lse=exp_lse, logits_soft_cap=cap)
    _check(out.cpu(), exp, out0, m, heads)
    ok = ~torch.isnan(exp_lse) & (exp_lse > -4e4)
    assert ok.any() and float((lse.cpu()[ok] - exp_lse[ok]).abs().max()) < 2e-2
    if cap == 1.0:   # the cap changes the result by far more than the tolerance: it was applied
        plain = oracle.sparse_attention(q, k, v, *sym, out=out0.clone())
        touched = _touched(m, heads, exp.shape)
        assert max_abs(plain[touched], exp[touched]) > 10 * MAX_ABS


def test_logits_soft_cap_packed_gqa_and_forward_options(dev):
    """The cap with the reference's grouped-query tiles (its own kernel instantiation), and set through
    the deprecated forward() (flashomni/attention.py:837-869), which stores it for later run() calls."""
    import flashomni_amd as fo
    H, Hkv, n = 4, 2, 384
    m = make_ragged_masks([n * (H // Hkv)], [n], Hkv, 0.8, 0.6, seed=23)   # symbols over packed rows x kv heads
    g = torch.Generator().manual_seed(23)
    q = (torch.randn(n, H, 128, generator=g) * 2).to(torch.bfloat16)
    k = torch.randn(n, Hkv, 128, generator=g).to(torch.bfloat16)
    v = torch.randn(n, Hkv, 128, generator=g).to(torch.bfloat16)
    t = lambda a: torch.from_numpy(a).to(dev)
    ip = torch.tensor([0, n], dtype=torch.int32, device=dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w.plan(ip, ip, H, Hkv, 128, q_data_type=torch.bfloat16)
    sym = (t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]))
    out0 = sentinel_like((n, H, 128), torch.bfloat16)
    exp = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"], m["keep_indptr"],
                                  [0, n], [0, n], out=out0.clone(), gqa_symbols="packed_tile", logits_soft_cap=2.0)
    got = w.forward(q.to(dev), k.to(dev), v.to(dev), *sym, logits_soft_cap=2.0)
    touched = (exp.view(torch.int16) != out0.view(torch.int16)).any(-1)
    assert touched.any()
    assert max_abs(got.cpu()[touched], exp[touched]) <= MAX_ABS and rel_l2(got.cpu()[touched], exp[touched]) <= REL_L2
    again = w.run(q.to(dev), k.to(dev), v.to(dev), *sym)    # the stored cap still applies
    assert torch.equal(again, got)


@pytest.mark.parametrize("seed", range(16))
def test_random_batches_all_options(dev, seed):
    """Seeded random batches over everything run() takes at once: 1-4 requests (now and then one without
    q rows or without keys), ungrouped heads or the reference's packed grouped-query tiles, both dtypes
    and kv layouts, the logits soft cap, lse.  Skipped rows keep their bytes; the rest within the path's
    tolerances of the oracle."""
    import flashomni_amd as fo
    rng = np.random.default_rng(5000 + seed)
    B = int(rng.integers(1, 5))
    ql = [int(rng.choice([1, 5, 127, 128, 129, 200, 384, 640, 1000])) for _ in range(B)]
    kl = [int(rng.choice([1, 64, 65, 128, 300, 513, 1024, 2048])) for _ in range(B)]
    if seed % 4 == 1:
        ql[int(rng.integers(0, B))] = 0
    if seed % 4 == 2:
        kl[int(rng.integers(0, B))] = 0
    if sum(ql) == 0:
        ql[0] = 130
    if sum(kl) == 0:
        kl[0] = 70
    hkv, group = int(rng.choice([1, 2, 3])), int(rng.choice([1, 1, 2, 4]))
    H = hkv * group
    dtype = torch.bfloat16 if seed % 2 == 0 else torch.float16
    layout = "NHD" if seed % 3 else "HND"
    cap = 4.0 if seed % 3 == 0 else 0.0
    pa, pk = float(rng.choice([0.3, 0.7, 1.0])), float(rng.choice([0.0, 0.1, 0.5, 1.0]))
    packed = group > 1
    m = make_ragged_masks([n * group for n in ql] if packed else ql, kl, hkv if packed else H, pa, pk, seed=5000 + seed)
    qo = np.concatenate([[0], np.cumsum(ql)]).astype(np.int32)
    g = torch.Generator().manual_seed(5000 + seed)
    nq, nk = sum(ql), sum(kl)
    q = torch.randn(nq, H, 128, generator=g).to(dtype)
    k = torch.randn(nk, hkv, 128, generator=g).to(dtype)
    v = torch.randn(nk, hkv, 128, generator=g).to(dtype)
    out0 = sentinel_like((nq, H, 128), dtype)
    t = lambda a: torch.from_numpy(a).to(dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(256 << 20, dtype=torch.uint8, device=dev), layout)
    w.plan(t(qo), t(m["kv_indptr"]), H, hkv, 128, q_data_type=dtype, logits_soft_cap=cap or None)
    kd, vd = k.to(dev), v.to(dev)
    if layout == "HND":
        kd, vd = kd.transpose(0, 1).contiguous(), vd.transpose(0, 1).contiguous()
    out = out0.clone().to(dev)
    _, lse = w.run(q.to(dev), kd, vd, t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]),
                   t(m["keep_indptr"]), out=out, return_lse=True)
    exp_lse = torch.full((nq, H), float("nan"))
    exp = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"], m["keep_indptr"], qo,
                                  m["kv_indptr"], out=out0.clone(), lse=exp_lse,
                                  gqa_symbols="packed_tile" if packed else "per_q_head", logits_soft_cap=cap)
    got = out.cpu()
    touched = ~torch.isnan(exp_lse)                     # [token, head]: rows the oracle wrote
    assert torch.equal(got[~touched].view(torch.int16), out0[~touched].view(torch.int16))
    if touched.any():
        assert max_abs(got[touched], exp[touched]) <= MAX_ABS
        if float(exp[touched].float().norm()) > 0:
            assert rel_l2(got[touched], exp[touched]) <= REL_L2
        assert float((lse.cpu()[touched] - exp_lse[touched]).abs().max()) < 2e-2
