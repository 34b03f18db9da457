"""GPU parity of the six ``torch.ops.flashomni_kernels`` operators, called positionally in the order
the reference's Python modules use (flashomni/attention.py:81-138, flashomni/gemm.py:61-85,106-129,
flashomni/quantization.py:55-61,148-159), against the oracle."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from helpers import make_ragged_masks, max_abs, rel_l2, sentinel_like

pytestmark = pytest.mark.gpu


def _ops():
    import flashomni_amd  # noqa: F401
    return torch.ops.flashomni_kernels


def _plan(dev, m, heads, float_ws=None, kv_heads=None):
    """What the reference's wrapper does in __init__ and plan() (flashomni/attention.py:344-352,
    :535-606): workspaces, host indptrs, the plan operator."""
    k = _ops()
    float_ws = torch.empty(128 << 20, dtype=torch.uint8, device=dev) if float_ws is None else float_ws
    int_ws = torch.empty(8 << 20, dtype=torch.uint8, device=dev)
    pin_ws = torch.empty(8 << 20, dtype=torch.uint8, pin_memory=True)
    qo_h, kv_h = torch.from_numpy(m["qo_indptr"]), torch.from_numpy(m["kv_indptr"])
    kv_len = kv_h[1:] - kv_h[:-1]
    batch = qo_h.numel() - 1
    plan_info = k.batch_sparseFA_with_kv_plan.default(
        float_ws, int_ws, pin_ws, qo_h, kv_h, kv_len, int(qo_h[-1]), batch, heads, kv_heads or heads, 1, False, 128,
        128)
    return float_ws, int_ws, plan_info, qo_h.to(dev), kv_h.to(dev)


def _run(dev, state, q, k, v, m, o, lse=None, is_full=False, layout=0, symbols=None):
    float_ws, int_ws, plan_info, qo_d, kv_d = state
    t = lambda a: torch.from_numpy(a).to(dev)
    if symbols is None:
        symbols = (t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]))
    _ops().batch_sparseFA_with_ragged_kv_run.default(
        float_ws, int_ws, plan_info, q, k, v, symbols[0], symbols[1], symbols[2], symbols[3], 128, 128, is_full,
        qo_d, kv_d, o, lse, 0, layout, None, None, None, 0.0, 128 ** -0.5, 1.0, 1.0 / 1e4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_attention_ops_ragged_batch(dev, dtype):
    heads = 3
    ql, kl = [300, 1, 128, 1000, 129], [77, 513, 128, 1100, 64]
    m = make_ragged_masks(ql, kl, heads, 0.75, 0.5, seed=21)
    g = torch.Generator().manual_seed(21)
    nq, nk = sum(ql), sum(kl)
    q, k, v = (torch.randn(n, heads, 128, generator=g).to(dtype) for n in (nq, nk, nk))
    state = _plan(dev, m, heads)
    exp_plan = oracle.prefill_plan(m["qo_indptr"], m["kv_indptr"], heads, heads, 128,
                                   torch.cuda.get_device_properties(dev).multi_processor_count,
                                   int_ws_bytes=8 << 20, float_ws_bytes=128 << 20)
    assert state[2].tolist() == list(exp_plan["plan_info"])
    out0 = sentinel_like((nq, heads, 128), dtype)
    o = out0.clone().to(dev)
    lse = torch.full((nq, heads), float("nan"), device=dev)
    _run(dev, state, q.to(dev), k.to(dev), v.to(dev), m, o, lse)
    exp_lse = torch.full((nq, heads), float("nan"))
    exp = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"],
                                  m["keep_indptr"], m["qo_indptr"], m["kv_indptr"], out=out0.clone(), lse=exp_lse)
    o = o.cpu()
    touched = (exp.view(torch.int16) != out0.view(torch.int16)).any(-1)
    assert torch.equal(o[~touched].view(torch.int16), out0[~touched].view(torch.int16))
    assert max_abs(o[touched], exp[touched]) <= 2e-2 and rel_l2(o[touched], exp[touched]) <= 1e-2
    ok = ~torch.isnan(exp_lse)
    assert torch.equal(torch.isnan(lse.cpu()), ~ok)
    assert float((lse.cpu()[ok] - exp_lse[ok]).abs().max()) < 2e-2


def test_attention_ops_grouped_query(dev):
    """num_kv_heads < num_qo_heads through the operators: the symbols are the reference's, one bit per
    (tile of 128 packed (token, q head) rows, kv head) (prefill.cuh:410-413, 1283-1290)."""
    hq, hkv = 8, 2
    ql, kl = [200, 129], [300, 64]
    m = make_ragged_masks([n * (hq // hkv) for n in ql], kl, hkv, 0.7, 0.5, seed=24)
    m["qo_indptr"] = np.concatenate([[0], np.cumsum(ql)]).astype(np.int32)
    g = torch.Generator().manual_seed(24)
    nq, nk = sum(ql), sum(kl)
    q = torch.randn(nq, hq, 128, generator=g).to(torch.bfloat16)
    k, v = (torch.randn(nk, hkv, 128, generator=g).to(torch.bfloat16) for _ in range(2))
    state = _plan(dev, m, hq, kv_heads=hkv)
    out0 = sentinel_like((nq, hq, 128), torch.bfloat16)
    o = out0.clone().to(dev)
    _run(dev, state, q.to(dev), k.to(dev), v.to(dev), m, o)
    exp = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"], m["keep_indptr"],
                                  m["qo_indptr"], m["kv_indptr"], out=out0.clone(), gqa_symbols="packed_tile")
    o = o.cpu()
    touched = (exp.view(torch.int16) != out0.view(torch.int16)).any(-1)
    assert touched.any() and not touched.all()
    assert torch.equal(o[~touched].view(torch.int16), out0[~touched].view(torch.int16))
    assert max_abs(o[touched], exp[touched]) <= 2e-2 and rel_l2(o[touched], exp[touched]) <= 1e-2


def test_attention_ops_hnd_and_is_full(dev):
    heads = 2
    m = make_ragged_masks([384], [640], heads, seed=22)
    g = torch.Generator().manual_seed(22)
    q, k, v = (torch.randn(n, heads, 128, generator=g).to(torch.bfloat16) for n in (384, 640, 640))
    state = _plan(dev, m, heads)
    o = torch.zeros(384, heads, 128, dtype=torch.bfloat16, device=dev)
    _run(dev, state, q.to(dev), k.to(dev).transpose(0, 1).contiguous(), v.to(dev).transpose(0, 1).contiguous(),
         m, o, is_full=True, layout=1, symbols=(None, None, None, None))
    exp = torch.nn.functional.scaled_dot_product_attention(
        q.float().transpose(0, 1), k.float().transpose(0, 1), v.float().transpose(0, 1)).transpose(0, 1)
    assert max_abs(o.cpu(), exp) <= 2e-2 and rel_l2(o.cpu(), exp) <= 1e-2


def test_attention_run_without_plan_is_refused(dev):
    heads = 2
    m = make_ragged_masks([256], [256], heads, seed=23)
    state = list(_plan(dev, m, heads))
    state[1] = torch.empty(8 << 20, dtype=torch.uint8, device=dev)   # an int workspace nothing was planned into
    q = torch.zeros(256, heads, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="no plan was made"):
        _run(dev, tuple(state), q, q, q, m, torch.zeros_like(q))
    state = _plan(dev, m, heads)
    with pytest.raises(RuntimeError, match="non-causal"):
        float_ws, int_ws, plan_info, qo_d, kv_d = state
        _ops().batch_sparseFA_with_ragged_kv_run.default(
            float_ws, int_ws, plan_info, q, q, q, None, None, None, None, 128, 128, True, qo_d, kv_d,
            torch.zeros_like(q), None, 1, 0, None, None, None, 0.0, 0.1, 1.0, 1e-4)


def test_attention_run_checks_the_plan_vector_and_plans_go_with_their_workspace(dev):
    """run() finds its plan by the int workspace: the plan vector the caller passes must be the one
    that plan call returned, and a plan is dropped when its workspace is freed (a later tensor at the
    same address must not find it)."""
    import gc
    from flashomni_amd import ops
    heads = 2
    m = make_ragged_masks([256], [256], heads, seed=25)
    float_ws, int_ws, plan_info, qo_d, kv_d = _plan(dev, m, heads)
    q = torch.zeros(256, heads, 128, dtype=torch.bfloat16, device=dev)
    _run(dev, (float_ws, int_ws, plan_info, qo_d, kv_d), q, q, q, m, torch.zeros_like(q))
    other = plan_info.clone()
    other[3] += 1
    with pytest.raises(RuntimeError, match="plan_info_vec is not the plan"):
        _run(dev, (float_ws, int_ws, other, qo_d, kv_d), q, q, q, m, torch.zeros_like(q))
    with pytest.raises(RuntimeError, match="planned number of heads"):
        q3 = torch.zeros(256, heads + 1, 128, dtype=torch.bfloat16, device=dev)
        _run(dev, (float_ws, int_ws, plan_info, qo_d, kv_d), q3, q, q, m, torch.zeros_like(q3))
    key = (dev.index, int_ws.data_ptr())
    assert key in ops._plans
    del int_ws
    gc.collect()
    assert key not in ops._plans


def test_symbols_rewritten_in_place_are_decoded_again(dev):
    """The symbol buffers are rewritten through the C ABI (a writer torch does not see: the tensors'
    version counters do not move); both the operator and the wrapper must run the new symbols."""
    import flashomni_amd as fo
    from flashomni_amd import _lib
    heads = 2
    ma = make_ragged_masks([512], [512], heads, 0.8, 0.6, seed=24)
    mb = make_ragged_masks([512], [512], heads, 0.5, 0.3, seed=25)
    g = torch.Generator().manual_seed(24)
    q, k, v = (torch.randn(512, heads, 128, generator=g).to(torch.bfloat16) for _ in range(3))
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    t = lambda a: torch.from_numpy(a).to(dev)
    info, keep = t(ma["packed_info"]).clone(), t(ma["packed_keep"]).clone()
    ip, kp = t(ma["info_indptr"]), t(ma["keep_indptr"])
    flags_b = t(np.concatenate([x.reshape(-1) for x in mb["info"]]).astype(np.uint8))
    keep_b = t(np.concatenate([x.reshape(-1) for x in mb["keep"]]).astype(np.uint8))
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w.plan(t(ma["qo_indptr"]), t(ma["kv_indptr"]), heads, heads, 128, q_data_type=torch.bfloat16)
    state = _plan(dev, ma, heads)

    def both(out0):
        o_w, o_op = out0.clone().to(dev), out0.clone().to(dev)
        w.run(qd, kd, vd, info, keep, ip, kp, out=o_w)
        _run(dev, state, qd, kd, vd, ma, o_op, symbols=(info, keep, ip, kp))
        return o_w.cpu(), o_op.cpu()

    out0 = sentinel_like((512, heads, 128), torch.bfloat16)
    exp_a = oracle.sparse_attention(q, k, v, ma["packed_info"], ma["packed_keep"], ma["info_indptr"],
                                    ma["keep_indptr"], ma["qo_indptr"], ma["kv_indptr"], out=out0.clone())
    for got in both(out0):
        assert max_abs(got, exp_a) <= 2e-2
    versions = (info._version, keep._version)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    L = _lib.lib()
    _lib.check(L.fo_packbits(flags_b.data_ptr(), flags_b.numel(), 1, info.data_ptr(), stream))
    _lib.check(L.fo_packbits(keep_b.data_ptr(), keep_b.numel(), 1, keep.data_ptr(), stream))
    assert (info._version, keep._version) == versions
    assert np.array_equal(info.cpu().numpy(), mb["packed_info"])
    exp_b = oracle.sparse_attention(q, k, v, mb["packed_info"], mb["packed_keep"], mb["info_indptr"],
                                    mb["keep_indptr"], mb["qo_indptr"], mb["kv_indptr"], out=out0.clone())
    for got in both(out0):
        touched = (exp_b.view(torch.int16) != out0.view(torch.int16)).any(-1)
        assert torch.equal(got[~touched].view(torch.int16), out0[~touched].view(torch.int16))
        assert max_abs(got[touched], exp_b[touched]) <= 2e-2
    # the opt-in: with reuse_decoded the caller vouches for unchanged symbols and gets the old list
    _lib.check(L.fo_packbits(t(np.concatenate([x.reshape(-1) for x in ma["keep"]]).astype(np.uint8)).data_ptr(),
                             keep_b.numel(), 1, keep.data_ptr(), stream))
    o_reuse = out0.clone().to(dev)
    w.run(qd, kd, vd, info, keep, ip, kp, out=o_reuse, reuse_decoded=True)
    touched = (exp_b.view(torch.int16) != out0.view(torch.int16)).any(-1)
    assert max_abs(o_reuse.cpu()[touched], exp_b[touched]) <= 2e-2


def test_attention_ops_logits_soft_cap(dev):
    """The run operator's logits_soft_cap argument (csrc/batch_sparseFA.cu:67-201 passes it to the
    variant, variants.cuh:43-56): equal to the wrapper planned with the same cap, and within the path's
    tolerances of the oracle."""
    import flashomni_amd as fo
    heads = 2
    m = make_ragged_masks([384, 130], [500, 256], heads, 0.8, 0.6, seed=33)
    g = torch.Generator().manual_seed(33)
    nq, nk = 514, 756
    q = (torch.randn(nq, heads, 128, generator=g) * 2).to(torch.bfloat16)
    k, v = (torch.randn(nk, heads, 128, generator=g).to(torch.bfloat16) for _ in range(2))
    state = _plan(dev, m, heads)
    float_ws, int_ws, plan_info, qo_d, kv_d = state
    t = lambda a: torch.from_numpy(a).to(dev)
    sym = (t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]))
    out0 = sentinel_like((nq, heads, 128), torch.bfloat16)
    o = out0.clone().to(dev)
    _ops().batch_sparseFA_with_ragged_kv_run.default(
        float_ws, int_ws, plan_info, q.to(dev), k.to(dev), v.to(dev), *sym, 128, 128, False,
        qo_d, kv_d, o, None, 0, 0, None, None, None, 3.0, 128 ** -0.5, 1.0, 1.0 / 1e4)
    exp = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"], m["keep_indptr"],
                                  m["qo_indptr"], m["kv_indptr"], out=out0.clone(), logits_soft_cap=3.0)
    touched = (exp.view(torch.int16) != out0.view(torch.int16)).any(-1)
    got = o.cpu()
    assert torch.equal(got[~touched].view(torch.int16), out0[~touched].view(torch.int16))
    assert max_abs(got[touched], exp[touched]) <= 2e-2 and rel_l2(got[touched], exp[touched]) <= 1e-2
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w.plan(t(m["qo_indptr"]), t(m["kv_indptr"]), heads, heads, 128, q_data_type=torch.bfloat16, logits_soft_cap=3.0)
    o_w = out0.clone().to(dev)
    w.run(q.to(dev), k.to(dev), v.to(dev), *sym, out=o_w)
    assert torch.equal(o_w.cpu().view(torch.int16), got.view(torch.int16))


def test_reuse_decoded_from_another_stream_waits_once_per_decode(dev):
    """A list decoded on a side stream and run from the current one: the first run waits for the
    decode, later ones on the same stream are behind it already (no further event), and a new decode
    is waited for again.  Each result is the oracle's for the symbols of its decode."""
    import flashomni_amd as fo
    heads = 2
    ma = make_ragged_masks([384], [384], heads, 0.7, 0.6, seed=5)
    mb = make_ragged_masks([384], [384], heads, 0.7, 0.6, seed=6)
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(384, heads, 128, generator=g).to(torch.bfloat16) for _ in range(3))
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    t = lambda a: torch.from_numpy(a).to(dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    w.plan(t(ma["qo_indptr"]), t(ma["kv_indptr"]), heads, heads, 128, q_data_type=torch.bfloat16)
    side = torch.cuda.Stream(device=dev)
    out0 = sentinel_like((384, heads, 128), torch.bfloat16)
    for m in (ma, mb):
        sym = (t(m["packed_info"]), t(m["packed_keep"]), t(m["info_indptr"]), t(m["keep_indptr"]))
        exp = oracle.sparse_attention(q, k, v, m["packed_info"], m["packed_keep"], m["info_indptr"],
                                      m["keep_indptr"], m["qo_indptr"], m["kv_indptr"], out=out0.clone())
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            # a long fill ahead of the decode, so that a run that did not wait would read the old list
            torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
            w.decode(*sym)
        assert w._planned.decoded[2] == []
        for rep in range(3):
            o = out0.clone().to(dev)
            w.run(qd, kd, vd, *sym, out=o, reuse_decoded=True)
            assert w._planned.decoded[2] == [torch.cuda.current_stream(dev)]
            touched = (exp.view(torch.int16) != out0.view(torch.int16)).any(-1)
            got = o.cpu()
            assert torch.equal(got[~touched].view(torch.int16), out0[~touched].view(torch.int16))
            assert max_abs(got[touched], exp[touched]) <= 2e-2


def test_plan_helpers_at_config0(dev):
    """plan() leaves the reference's bit-count indptrs (flashomni/attention.py:625-642)."""
    import flashomni_amd as fo
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(128 << 20, dtype=torch.uint8, device=dev))
    ip = torch.tensor([0, 4608], dtype=torch.int32, device=dev)
    w.plan(ip, ip, 24, 24, 128, q_data_type=torch.bfloat16)
    assert w._sparse_info_indptr_base.tolist() == [0, 864]
    assert w._sparse_kv_info_indptr_base.tolist() == [0, 31104]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gemm_ops(dev, dtype):
    heads, M, hid = 4, 128 * 5 + 80, 512
    m = make_ragged_masks([M], [M], heads, 0.6, 0.5, seed=31)
    g = torch.Generator().manual_seed(31)
    x = torch.randn(1, M, hid, generator=g).to(dtype)
    w = (torch.randn(hid, hid, generator=g) * 0.05).to(dtype)
    b = (torch.randn(hid, generator=g) * 0.05).to(dtype)
    info, ip = torch.from_numpy(m["packed_info"]), torch.from_numpy(m["info_indptr"])
    k = _ops()
    y0 = sentinel_like((1, M, hid), dtype)
    y = y0.clone().to(dev)
    # flashomni/gemm.py:74-85: (A, B, out, bias, sparse_q_size, num_qo_heads, info, indptr, num_text_tokens, is_full)
    k.flashomni_gemm.default(x.to(dev), w.to(dev), y, b.to(dev), 128, heads, info.to(dev), ip.to(dev), 0, False)
    exp = oracle.gemm_q(x, w, heads, info, ip, 0, b, out=y0.clone())
    y = y.cpu()
    touched = (exp.view(torch.int16) != y0.view(torch.int16))
    assert torch.equal(y[~touched].view(torch.int16), y0[~touched].view(torch.int16))
    assert max_abs(y, exp) <= 2e-2
    # flashomni/gemm.py:118-129, two-call protocol of benchmark/test_flashomni_gemm_o.py:72-80
    cache = torch.empty(1, M, hid, dtype=dtype, device=dev)
    k.flashomni_gemm_reduction.default(x.to(dev), w.to(dev), cache, b.to(dev), 128, heads, info.to(dev),
                                       ip.to(dev), 0, True)
    exp_cache = oracle.gemm_o(x, w, heads, info, ip, 0, bias=b, is_for_cache=True)
    assert max_abs(cache.cpu(), exp_cache) <= 2e-2
    final = torch.empty(1, M, hid, dtype=dtype, device=dev)
    k.flashomni_gemm_reduction.default(x.to(dev), w.to(dev), final, cache, 128, heads, info.to(dev),
                                       ip.to(dev), 0, False)
    dense = torch.nn.functional.linear(x.float(), w.float(), b.float())
    assert max_abs(final.cpu(), dense) <= 4e-2
    with pytest.raises(RuntimeError, match="Token sizes must match"):
        k.flashomni_gemm.default(x.to(dev), w.to(dev), torch.empty(1, M + 1, hid, dtype=dtype, device=dev), None,
                                 128, heads, None, None, 0, True)


def test_packbits_ops(dev):
    k = _ops()
    # docstring vectors of flashomni/quantization.py:90-93 and :133-138
    x = torch.tensor([1, 0, 1, 1, 0, 0, 1, 1], dtype=torch.bool, device=dev)
    y = torch.empty(1, dtype=torch.uint8, device=dev)
    k.packbits.default(x, "big", y)
    assert y.tolist() == [0b10110011]
    x = torch.tensor([1, 0, 1, 1, 0, 0, 1, 1, 1, 0, 1], dtype=torch.bool, device=dev)
    ip = torch.tensor([0, 4, 7, 11], dtype=torch.int32, device=dev)
    op = torch.tensor([0, 1, 2, 3], dtype=torch.int32, device=dev)
    y = torch.empty(3, dtype=torch.uint8, device=dev)
    k.segment_packbits.default(x, ip, op, "big", y)
    assert y.tolist() == [0b10110000, 0b100000, 0b11010000]
    rng = np.random.default_rng(5)
    bits = rng.random(10007) < 0.4
    y = torch.empty((10007 + 7) // 8, dtype=torch.uint8, device=dev)
    for order in ("big", "little"):
        k.packbits.default(torch.from_numpy(bits).to(dev), order, y)
        assert np.array_equal(y.cpu().numpy(), np.packbits(bits, bitorder=order))
