"""run() and the GEMMs under HIP graph capture (the reference declares run() capturable,
flashomni/attention.py:140-141): a captured layer pass must give, on every replay, what the same
calls give eagerly on the inputs of that moment, including symbols rewritten in place between
replays."""
import numpy as np
import pytest
import torch

from helpers import make_ragged_masks

pytestmark = pytest.mark.gpu


def test_captured_layer_pass_replays(dev):
    import flashomni_amd as fo
    H, hidden = 4, 512
    ql = [640, 300]
    nnz = sum(ql)
    g = torch.Generator().manual_seed(5)
    rnd = lambda *s: torch.randn(*s, generator=g)
    x = rnd(1, nnz, hidden).to(torch.bfloat16).to(dev)
    wq = (rnd(hidden, hidden) * 0.05).to(torch.bfloat16).to(dev)
    bq = (rnd(hidden) * 0.05).to(torch.bfloat16).to(dev)
    wo = (rnd(hidden, hidden) * 0.05).to(torch.bfloat16).to(dev)
    k = rnd(nnz, H, 128).to(torch.bfloat16).to(dev)
    v = rnd(nnz, H, 128).to(torch.bfloat16).to(dev)

    def symbols(seed):
        m = make_ragged_masks(ql, ql, H, 0.7, 0.5, seed=seed)
        return [torch.from_numpy(m[n]) for n in ("packed_info", "packed_keep", "info_indptr", "keep_indptr")]

    info, kv_info, info_ip, kv_ip = [t.to(dev) for t in symbols(1)]
    # the GEMMs see the two requests as one batch entry of nnz rows: their symbols index the
    # 128-row blocks of that entry, so give them a single-request packing of the same size
    n_blk = sum(-(-l // 128) for l in ql)
    gemm_bits = torch.from_numpy((np.random.default_rng(2).random(n_blk * H) < 0.7))
    gemm_info = fo.packbits(gemm_bits.to(dev), "little")
    gemm_ip = torch.tensor([0, gemm_info.numel()], dtype=torch.int32, device=dev)

    ws = torch.empty(32 << 20, dtype=torch.uint8, device=dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(ws)
    indptr = torch.tensor([0, ql[0], nnz], dtype=torch.int32)
    w.plan(indptr, indptr, H, H, 128, q_data_type=torch.bfloat16)

    q_buf = torch.zeros(1, nnz, hidden, dtype=torch.bfloat16, device=dev)
    o_buf = torch.zeros(nnz, H, 128, dtype=torch.bfloat16, device=dev)
    y_buf = torch.zeros(1, nnz, hidden, dtype=torch.bfloat16, device=dev)

    def layer_pass(q_out, o_out):
        fo.flashomni_gemm(x, wq, H, gemm_info, gemm_ip, 0, bq, out=q_out)
        w.run(q_out.view(nnz, H, 128), k, v, info, kv_info, info_ip, kv_ip, out=o_out)
        return fo.flashomni_gemm_reduction(o_out.view(1, nnz, hidden), wo, H, gemm_info, gemm_ip, 0,
                                           bias=None, is_for_cache=False)

    # warm up on a side stream, then capture
    s = torch.cuda.Stream(device=dev)
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        layer_pass(q_buf, o_buf)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_graph = layer_pass(q_buf, o_buf)
    for replay in range(4):
        # new activations and, from the second replay on, new attention symbols, written in place
        x.copy_(rnd(1, nnz, hidden).to(torch.bfloat16))
        if replay >= 1:
            for dst, src in zip((info, kv_info), symbols(10 + replay)[:2]):
                dst.copy_(src)
        q_buf.zero_(); o_buf.zero_()
        graph.replay()
        torch.cuda.synchronize()
        got = (q_buf.clone(), o_buf.clone(), y_graph.clone())
        # the same pass eagerly, into fresh buffers, with program work and a sync in between
        q_ref = torch.zeros_like(q_buf); o_ref = torch.zeros_like(o_buf)
        y_ref = layer_pass(q_ref, o_ref)
        torch.cuda.synchronize()
        for name, a, b in zip(("gemm_q", "attention", "gemm_o"), got, (q_ref, o_ref, y_ref)):
            assert torch.equal(a, b), "replay %d: %s differs from the eager pass" % (replay, name)


def test_captured_long_gemm_o_replays(dev):
    """A GEMM-O launch long enough to hand out its work items through cursors (four items or more per CU):
    the kernel that clears the cursors is captured with it, so every replay starts from zero.  Flags and
    activations are rewritten in place between replays; each replay equals the eager call of that moment."""
    import flashomni_amd as fo
    m, n, heads = 22016, 3072, 24
    g = torch.Generator(device=dev).manual_seed(9)
    x = torch.randn(1, m, n, generator=g, device=dev).to(torch.bfloat16)
    w = (torch.randn(n, n, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    b = (torch.randn(n, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    rng = np.random.default_rng(3)
    bits = lambda: torch.from_numpy(rng.random((m // 128) * heads) < 0.3)
    info = fo.packbits(bits().to(dev), "little")
    ip = torch.tensor([0, info.numel()], dtype=torch.int32, device=dev)

    def two_passes():
        cache = fo.flashomni_gemm_reduction(x, w, heads, info, ip, 0, bias=b, is_for_cache=True)
        return cache, fo.flashomni_gemm_reduction(x, w, heads, info, ip, 0, bias=cache, is_for_cache=False)

    s = torch.cuda.Stream(device=dev)
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        two_passes()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cache_g, final_g = two_passes()
    for replay in range(3):
        x.copy_(torch.randn(1, m, n, generator=g, device=dev).to(torch.bfloat16))
        if replay >= 1:
            info.copy_(fo.packbits(bits().to(dev), "little"))
        graph.replay()
        torch.cuda.synchronize()
        got = (cache_g.clone(), final_g.clone())
        ref = two_passes()
        torch.cuda.synchronize()
        for name, a, r in zip(("cache pass", "final pass"), got, ref):
            assert torch.equal(a, r), "replay %d: %s differs from the eager call" % (replay, name)


def test_graph_captured_on_a_warm_stream_survives_workspace_growth(dev):
    """GEMM-Q keeps its tile list in a scratch buffer cached per stream.  A graph captured on a stream
    that already ran the GEMM eagerly must not record that cached buffer: a later, larger eager GEMM on
    the same stream replaces it, and a replay would then write its list into memory that may belong to
    someone else.  Capture on the warm stream, grow the scratch eagerly on it, replay, compare."""
    import flashomni_amd as fo
    from flashomni_amd import gemm as gemm_mod
    heads, hidden = 4, 512
    g = torch.Generator(device=dev).manual_seed(17)
    rng = np.random.default_rng(17)

    def problem(m):
        x = torch.randn(1, m, hidden, generator=g, device=dev).to(torch.bfloat16)
        info = fo.packbits(torch.from_numpy(rng.random(-(-m // 128) * heads) < 0.6).to(dev), "little")
        ip = torch.tensor([0, info.numel()], dtype=torch.int32, device=dev)
        return x, info, ip

    w = (torch.randn(hidden, hidden, generator=g, device=dev) * 0.05).to(torch.bfloat16)
    # (large enough that the tile list is built by the list kernel into the scratch buffer)
    x, info, ip = problem(128 * 300)
    out = torch.zeros(1, x.size(1), hidden, dtype=torch.bfloat16, device=dev)
    s = torch.cuda.Stream(device=dev)
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fo.flashomni_gemm(x, w, heads, info, ip, 0, None, out=out)   # eager warm-up on s
    s.synchronize()
    eager_bufs = {b.data_ptr() for b in gemm_mod._workspaces[(dev.index, s.cuda_stream)]}
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=s):
        fo.flashomni_gemm(x, w, heads, info, ip, 0, None, out=out)
    # a much larger GEMM on the same stream: the stream's scratch buffer is replaced
    xb, infob, ipb = problem(128 * 3000)
    with torch.cuda.stream(s):
        big = fo.flashomni_gemm(xb, w, heads, infob, ipb, 0, None)
    s.synchronize()
    bufs = gemm_mod._workspaces[(dev.index, s.cuda_stream)]
    assert len(bufs) >= 2 and eager_bufs <= {b.data_ptr() for b in bufs}, "superseded scratch must stay alive"
    del big, xb
    torch.cuda.empty_cache()
    junk = [torch.full((1 << 20,), 0x5a, dtype=torch.uint8, device=dev) for _ in range(8)]  # reuse freed memory
    for replay in range(3):
        x.copy_(torch.randn(1, x.size(1), hidden, generator=g, device=dev).to(torch.bfloat16))
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        ref = torch.zeros_like(out)
        fo.flashomni_gemm(x, w, heads, info, ip, 0, None, out=ref)
        torch.cuda.synchronize()
        assert torch.equal(out, ref), "replay %d differs from the eager call" % replay
        assert all(bool((j == 0x5a).all()) for j in junk), "a replay wrote outside its own scratch"
