#!/usr/bin/env python3
"""Benchmark of the sparse-attention hot path on one MI355X.

One *step* is one sparse pass of a FLUX-shaped layer (configs 0-2 of the baseline):
GEMM-Q over the flagged (token-block, head) tiles -> symbol decode + block-sparse FlashAttention
-> GEMM-O that adds the non-cached heads to the cached partial.  ``value`` is the effective
TFLOP/s of that chain, counting only computed blocks / tiles / head slices.

The JSON line also carries
  * ``kernels``: per-kernel latency and effective TFLOP/s (or GB/s) for every config, each as a
    fraction of the MI355X peak that bounds it,
  * ``roofline``: the dominant kernel (sparse FlashAttention at the FLUX shape) measured with HIP
    events on the launch stream,
  * ``cpu_baseline``: the fp32 CPU path (the oracle) timed on this box's host cores: the whole FLUX
    layer, and under ``c3`` / ``c4`` a sample of the big configs' attention rows and token blocks
    with the extrapolation to the whole config labelled as such.

Every attention config also carries ``run_dropin``: the reference's call sequence
``wrapper.run(q, k, v, sparse_info, sparse_kv_info, indptrs)`` with a fresh decode in every call.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs 0,1,2,3,4] [--no-cpu]
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "hbm_traffic_flux_layer_c0_c1_c2.txt")
SETTLE_MS = 150.0    # load applied before any timing: an idle device's clocks take ~100 ms to ramp
PEAK_BF16 = 2516.6   # TFLOP/s dense
PEAK_FP8 = 5033.2
PEAK_HBM = 8000.0    # GB/s


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def kernel_source_hash():
    import hashlib
    with open(os.path.join(ROOT, "flashomni_amd", "csrc", "sparse_fa.hip"), "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:16]


def traffic_from_profile():
    """HBM bytes per sparse-FA launch at config 0, as recorded in the committed rocprofv3 summary
    (line ``traffic_bytes_per_launch <kernel> = <bytes>``), and whether that summary was taken from the
    kernel source this run uses (line ``kernel_source_sha256 sparse_fa.hip = <first 16 hex digits>``).
    (None, reason) when the summary has no such line or describes another version of the kernel: a
    counter reading of other code is not this run's traffic."""
    value = recorded = None
    try:
        for line in open(TRAFFIC_PROFILE):
            if line.startswith("traffic_bytes_per_launch sparse_fa_kernel<bf16>"):
                value = float(line.split("=")[1].split()[0])
            if line.startswith("kernel_source_sha256 sparse_fa.hip"):
                recorded = line.split("=")[1].split()[0]
    except OSError:
        return None, "no counter summary"
    if value is None:
        return None, "no counter summary"
    if recorded != kernel_source_hash():
        return None, "the counter summary was taken from another version of the kernel source"
    return value, "current"


def time_gpu(fn, iters, warmup):
    """Average milliseconds per call, HIP events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / iters


def entry(ms, flops=None, nbytes=None, peak=None):
    d = {"ms": round(ms, 5)}
    if flops is not None:
        d["tflops"] = round(flops / (ms * 1e-3) / 1e12, 2)
        d["frac_of_peak"] = round(d["tflops"] / (peak or PEAK_BF16), 4)
    if nbytes is not None:
        d["gbps"] = round(nbytes / (ms * 1e-3) / 1e9, 2)
        d["frac_of_peak"] = round(d["gbps"] / PEAK_HBM, 4)
    return d


class FluxLayer:
    """Configs 0-2 on the device + the wrappers needed to run the chain."""

    def __init__(self, dev):
        import flashomni_amd as fo
        from flashomni_amd.workloads import make_workload
        self.fo = fo
        self.w0, self.w1, self.w2 = make_workload(0), make_workload(1), make_workload(2)
        d = lambda t: t.to(dev)
        self.q, self.k, self.v = (d(self.w0.tensors[n]) for n in "qkv")
        self.x, self.wq, self.bq = d(self.w1.tensors["x"]), d(self.w1.tensors["w"]), d(self.w1.tensors["bias"])
        self.a, self.wo, self.bo = d(self.w2.tensors["a"]), d(self.w2.tensors["w"]), d(self.w2.tensors["bias"])
        self.info, self.kv_info = d(self.w0.packed_info), d(self.w0.packed_kv_info)
        self.info_ip, self.kv_ip = d(self.w0.info_indptr), d(self.w0.kv_info_indptr)
        self.ws = torch.empty(128 << 20, dtype=torch.uint8, device=dev)
        self.wrapper = fo.BatchFlashOmniFAWithRaggedKVWrapper(self.ws)
        self.wrapper.plan(self.w0.qo_indptr, self.w0.kv_indptr, 24, 24, 128, q_data_type=torch.bfloat16)
        self.side = torch.cuda.Stream(device=dev)
        self.out_q = torch.zeros(1, 4608, 3072, dtype=torch.bfloat16, device=dev)
        self.out_fa = torch.zeros(4608, 24, 128, dtype=torch.bfloat16, device=dev)
        self.cache = fo.flashomni_gemm_reduction(self.a, self.wo, 24, self.info, self.info_ip, 0,
                                                 bias=self.bo, is_for_cache=True)

    def gemm_q(self):
        return self.fo.flashomni_gemm(self.x, self.wq, 24, self.info, self.info_ip, 0, self.bq,
                                      out=self.out_q)

    def decode(self):
        return self.wrapper.decode(self.info, self.kv_info, self.info_ip, self.kv_ip)

    def attention(self, fresh_decode=True):
        """fresh_decode=False: run the list the last decode() left (ordered after it across streams)."""
        return self.wrapper.run(self.q, self.k, self.v, self.info, self.kv_info, self.info_ip,
                                self.kv_ip, out=self.out_fa, reuse_decoded=not fresh_decode)

    def gemm_o_cache(self):
        return self.fo.flashomni_gemm_reduction(self.a, self.wo, 24, self.info, self.info_ip, 0,
                                                bias=self.bo, is_for_cache=True)

    def gemm_o_final(self):
        return self.fo.flashomni_gemm_reduction(self.a, self.wo, 24, self.info, self.info_ip, 0,
                                                bias=self.cache, is_for_cache=False)

    def step(self):
        """One sparse pass of the layer.  The decode of the step's symbols does not depend on the
        Q projection, so it runs on a second stream (default priority) beside GEMM-Q; attention
        waits for both."""
        cur = torch.cuda.current_stream()
        self.side.wait_stream(cur)      # the work list is free once the previous attention is done
        with torch.cuda.stream(self.side):
            self.decode()               # a fresh decode every step
        self.gemm_q()
        cur.wait_stream(self.side)
        self.attention(fresh_decode=False)
        return self.gemm_o_final()

    def step_dropin(self):
        """The same pass as the reference's call sequence on one stream: flashomni_gemm, then
        wrapper.run(q, k, v, symbols...) (which decodes the symbols itself), then
        flashomni_gemm_reduction."""
        self.gemm_q()
        self.attention(fresh_decode=True)
        return self.gemm_o_final()

    def chain_flops(self):
        return self.w1.gemm_q_flops() + self.w0.attention_flops() + self.w2.gemm_o_flops(False)


def captured_step_ms(layer, dev, iters, warmup):
    """The layer's two-stream step captured as one HIP graph: every one of three replays (eager work
    and a sync between them) must equal the eager step; then milliseconds per replay."""
    ref_o = layer.step().clone()
    torch.cuda.synchronize()
    cap = torch.cuda.Stream(device=dev)
    cap.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(cap):
        layer.step()  # (the stream's own scratch buffers exist before the capture)
    torch.cuda.current_stream().wait_stream(cap)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=cap):
        graph_o = layer.step()
    for rep in range(3):
        layer.out_q.zero_(); layer.out_fa.zero_()
        graph.replay()
        torch.cuda.synchronize()
        if not torch.equal(graph_o, ref_o):
            raise AssertionError("replay %d differs from the eager step" % rep)
    for _ in range(warmup):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        graph.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / iters


def bench_big_attention(dev, index, iters, warmup, with_cpu=False):
    """Configs 3 / 4 attention at full size (tensors drawn on the GPU: the CPU draw of 10^9 normals
    would dominate the run; masks are the seeded CPU ones).  with_cpu: also time the oracle on a sample
    of the same rows (second return value)."""
    import flashomni_amd as fo
    from flashomni_amd.workloads import make_workload
    wl = make_workload(index, tensors=False)
    s = wl.shape
    g = torch.Generator(device=dev).manual_seed(1000 + index)
    mk = lambda: torch.randn(s.seq, s.heads, 128, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    q, k, v = mk(), mk(), mk()
    ws = torch.empty(128 << 20, dtype=torch.uint8, device=dev)
    w = fo.BatchFlashOmniFAWithRaggedKVWrapper(ws)
    w.plan(wl.qo_indptr, wl.kv_indptr, s.heads, s.heads, 128, q_data_type=torch.bfloat16)
    args = [t.to(dev) for t in (wl.packed_info, wl.packed_kv_info, wl.info_indptr, wl.kv_info_indptr)]
    out = torch.zeros_like(q)

    res = {}
    ms = time_gpu(lambda: w.decode(*args), iters, warmup)
    rows, nnz = w._worklist.sizes()
    dec_bytes = wl.packed_info.numel() + wl.packed_kv_info.numel() + 4 * (4 * rows + 1 + nnz)
    res["decode"] = entry(ms, nbytes=dec_bytes)
    res["decode"]["rows"], res["decode"]["kv_blocks"] = rows, nnz
    ms = time_gpu(lambda: w.run(q, k, v, *args, out=out, reuse_decoded=True), iters, warmup)
    res["sparse_fa_bf16"] = entry(ms, flops=wl.attention_flops())
    res["sparse_fa_bf16"]["computed_blocks"] = wl.computed_blocks
    # the call a user of the reference makes: decode of the symbols + attention, every time
    ms = time_gpu(lambda: w.run(q, k, v, *args, out=out), iters, warmup)
    res["run_dropin"] = entry(ms, flops=wl.attention_flops())
    cpu = cpu_baseline_attention(wl, q.cpu(), k.cpu(), v.cpu()) if with_cpu else None
    if index == 4:
        # fp8 e4m3 Q.K^T (per-(head, 128-token block) absmax scales), bf16 P.V.  q as two e4m3 terms
        # (q + residual: the form that meets the fp8 accuracy contract) and as one term (faster, outside it)
        blocks = tuple(t.to(dev) for t in fo.token_blocks(wl.qo_indptr))
        ms_q = time_gpu(lambda: fo.quant_fp8_block(q, wl.qo_indptr, blocks=blocks), iters, warmup)
        res["quant_fp8"] = entry(ms_q, nbytes=3 * q.numel() + 4 * s.heads * s.n_blocks)
        ms_q = time_gpu(lambda: fo.quant_fp8_block(q, wl.qo_indptr, blocks=blocks, residual=True), iters, warmup)
        res["quant_fp8_two_term"] = entry(ms_q, nbytes=4 * q.numel() + 4 * s.heads * s.n_blocks)
        # context, not a product path: a device-to-device copy of the same tensor (what a kernel that
        # reads and writes streams reaches on this device)
        qc = torch.empty_like(q)
        res["device_copy_same_tensor"] = entry(time_gpu(lambda: qc.copy_(q), iters, warmup), nbytes=4 * q.numel())
        del qc
        q8, qs, q_lo = fo.quant_fp8_block(q, wl.qo_indptr, blocks=blocks, residual=True)
        k8, ks, k_lo = fo.quant_fp8_block(k, wl.kv_indptr, blocks=blocks, residual=True)
        w8 = fo.BatchFlashOmniFAWithRaggedKVWrapper(ws)
        w8.plan(wl.qo_indptr, wl.kv_indptr, s.heads, s.heads, 128, q_data_type=torch.float8_e4m3fn)
        out8 = torch.zeros_like(q)
        w8.decode(*args)
        w.run(q, k, v, *args, out=out)
        # two terms of q and of k (value + rounding residual under one scale): the form that meets the
        # fp8 accuracy contract of the whole chain; two terms of q only; one term each (fastest)
        for name, lo, klo, peak in (("sparse_fa_fp8qk", q_lo, k_lo, PEAK_BF16),
                                    ("sparse_fa_fp8qk_q_two_term", q_lo, None, PEAK_BF16),
                                    # one term: QK^T half at the fp8 peak, PV half at the bf16 peak
                                    ("sparse_fa_fp8qk_one_term", None, None, 2.0 / (1 / PEAK_FP8 + 1 / PEAK_BF16))):
            ms8 = time_gpu(lambda: w8.run(q8, k8, v, *args, out=out8, q_scale=qs, k_scale=ks, q_lo=lo,
                                          k_lo=klo, reuse_decoded=True), iters, warmup)
            res[name] = entry(ms8, flops=wl.attention_flops(), peak=peak)
            res[name]["frac_of_bf16_peak"] = round(res[name]["tflops"] / PEAK_BF16, 4)
            # error of the fp8 output against the bf16 kernel's output on the same inputs
            num = (out8.float() - out.float()).norm()
            res[name]["rel_l2_vs_bf16_kernel"] = round(float(num / out.float().norm()), 4)
        del q8, k8, out8, q_lo, k_lo
    del q, k, v, out
    torch.cuda.empty_cache()
    return res, cpu


def bench_big_gemms(dev, index, iters, warmup, with_cpu=False):
    import flashomni_amd as fo
    from flashomni_amd.workloads import make_workload
    wl = make_workload(index, tensors=False)
    s = wl.shape
    g = torch.Generator(device=dev).manual_seed(2000 + index)
    x = torch.randn(1, s.seq, s.hidden, generator=g, device=dev).to(torch.bfloat16)
    wq = (torch.randn(s.hidden, s.hidden, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    bq = (torch.randn(s.hidden, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    info, ip = wl.packed_info.to(dev), wl.info_indptr.to(dev)
    out = torch.zeros(1, s.seq, s.hidden, dtype=torch.bfloat16, device=dev)
    res = {}
    ms = time_gpu(lambda: fo.flashomni_gemm(x, wq, s.heads, info, ip, 0, bq, out=out), iters, warmup)
    res["gemm_q"] = entry(ms, flops=wl.gemm_q_flops())
    # the same projection with the fp8 quantisation of its result fused in (no 16-bit result written)
    q8 = torch.empty(1, s.seq, s.hidden, dtype=torch.float8_e4m3fn, device=dev)
    q8s = torch.empty(s.heads, s.n_blocks, dtype=torch.float32, device=dev)
    ms = time_gpu(lambda: fo.flashomni_gemm(x, wq, s.heads, info, ip, 0, bq, out=False, quant_out=(q8, q8s)),
                  iters, warmup)
    res["gemm_q_fused_fp8"] = entry(ms, flops=wl.gemm_q_flops())
    q8lo = torch.empty_like(q8)
    ms = time_gpu(lambda: fo.flashomni_gemm(x, wq, s.heads, info, ip, 0, bq, out=False, quant_out=(q8, q8s, q8lo)),
                  iters, warmup)
    res["gemm_q_fused_fp8_two_term"] = entry(ms, flops=wl.gemm_q_flops())
    del q8, q8s, q8lo
    ms = time_gpu(lambda: fo.flashomni_gemm_reduction(x, wq, s.heads, info, ip, 0, bias=bq,
                                                      is_for_cache=True), iters, warmup)
    res["gemm_o_cache"] = entry(ms, flops=wl.gemm_o_flops(True))
    cache = fo.flashomni_gemm_reduction(x, wq, s.heads, info, ip, 0, bias=bq, is_for_cache=True)
    ms = time_gpu(lambda: fo.flashomni_gemm_reduction(x, wq, s.heads, info, ip, 0, bias=cache,
                                                      is_for_cache=False), iters, warmup)
    res["gemm_o_final"] = entry(ms, flops=wl.gemm_o_flops(False))
    # context, not a product path: the vendor library's dense bf16 GEMM of the same shape on this device
    ms = time_gpu(lambda: torch.matmul(x[0], wq.t()), iters, warmup)
    res["vendor_dense_gemm_same_shape"] = entry(ms, flops=2.0 * s.seq * s.hidden * s.hidden)
    cpu = cpu_baseline_gemms(wl, x.cpu(), wq.cpu(), bq.cpu()) if with_cpu else None
    del x, wq, out, cache
    torch.cuda.empty_cache()
    return res, cpu


def bench_wan_chain(dev, iters, warmup):
    """Config 4 end to end: GEMM-Q (two-term fp8 result from its epilogue) -> two-term fp8 quantisation
    of K -> symbol decode + sparse FA (fp8 Q.K^T) -> GEMM-O final pass; and the same chain in bf16 without
    any quantisation.  K, V drawn directly (the chain of the task has no K/V projection)."""
    import flashomni_amd as fo
    from flashomni_amd.workloads import make_workload
    wl = make_workload(4, tensors=False)
    s = wl.shape
    g = torch.Generator(device=dev).manual_seed(3004)
    rnd = lambda *shape: torch.randn(*shape, generator=g, device=dev, dtype=torch.float32)
    x = rnd(1, s.seq, s.hidden).to(torch.bfloat16)
    wq = (rnd(s.hidden, s.hidden) * 0.02).to(torch.bfloat16)
    wo = (rnd(s.hidden, s.hidden) * 0.02).to(torch.bfloat16)
    bq = (rnd(s.hidden) * 0.02).to(torch.bfloat16)
    k = rnd(s.seq, s.heads, 128).to(torch.bfloat16)
    v = rnd(s.seq, s.heads, 128).to(torch.bfloat16)
    info, ip = wl.packed_info.to(dev), wl.info_indptr.to(dev)
    kv_info, kv_ip = wl.packed_kv_info.to(dev), wl.kv_info_indptr.to(dev)
    ws = torch.empty(128 << 20, dtype=torch.uint8, device=dev)
    w8 = fo.BatchFlashOmniFAWithRaggedKVWrapper(ws)
    w8.plan(wl.qo_indptr, wl.kv_indptr, s.heads, s.heads, 128, q_data_type=torch.float8_e4m3fn)
    w16 = fo.BatchFlashOmniFAWithRaggedKVWrapper(ws)
    w16.plan(wl.qo_indptr, wl.kv_indptr, s.heads, s.heads, 128, q_data_type=torch.bfloat16)
    blocks = tuple(t.to(dev) for t in fo.token_blocks(wl.kv_indptr))
    q8 = torch.zeros(1, s.seq, s.hidden, dtype=torch.float8_e4m3fn, device=dev)
    q8lo = torch.zeros(1, s.seq, s.hidden, dtype=torch.float8_e4m3fn, device=dev)
    q8s = torch.ones(s.heads, s.n_blocks, dtype=torch.float32, device=dev)
    q16 = torch.zeros(1, s.seq, s.hidden, dtype=torch.bfloat16, device=dev)
    o = torch.zeros(s.seq, s.heads, 128, dtype=torch.bfloat16, device=dev)
    cache = fo.flashomni_gemm_reduction(o.view(1, s.seq, s.hidden), wo, s.heads, info, ip, 0, bias=None,
                                        is_for_cache=True)

    # As in the FLUX step, what does not depend on the Q projection (the decode of the symbols; for fp8
    # also the quantisation of K) runs on a second stream (default priority) beside GEMM-Q.
    side = torch.cuda.Stream(device=dev)

    def chain_fp8():
        cur = torch.cuda.current_stream()
        side.wait_stream(cur)
        with torch.cuda.stream(side):
            w8.decode(info, kv_info, ip, kv_ip)
            k8, ks, k8lo = fo.quant_fp8_block(k, wl.kv_indptr, blocks=blocks, residual=True)
        fo.flashomni_gemm(x, wq, s.heads, info, ip, 0, bq, out=False, quant_out=(q8, q8s, q8lo))
        cur.wait_stream(side)
        for t in (k8, ks, k8lo):
            t.record_stream(cur)
        w8.run(q8.view(s.seq, s.heads, 128), k8, v, info, kv_info, ip, kv_ip, out=o, q_scale=q8s, k_scale=ks,
               q_lo=q8lo.view(s.seq, s.heads, 128), k_lo=k8lo, reuse_decoded=True)
        return fo.flashomni_gemm_reduction(o.view(1, s.seq, s.hidden), wo, s.heads, info, ip, 0, bias=cache,
                                           is_for_cache=False)

    def chain_bf16():
        cur = torch.cuda.current_stream()
        side.wait_stream(cur)
        with torch.cuda.stream(side):
            w16.decode(info, kv_info, ip, kv_ip)
        fo.flashomni_gemm(x, wq, s.heads, info, ip, 0, bq, out=q16)
        cur.wait_stream(side)
        w16.run(q16.view(s.seq, s.heads, 128), k, v, info, kv_info, ip, kv_ip, out=o, reuse_decoded=True)
        return fo.flashomni_gemm_reduction(o.view(1, s.seq, s.hidden), wo, s.heads, info, ip, 0, bias=cache,
                                           is_for_cache=False)

    flops = wl.gemm_q_flops() + wl.attention_flops() + wl.gemm_o_flops(False)
    res = {}
    y16 = chain_bf16().float()
    y8 = chain_fp8().float()
    res["chain_bf16"] = entry(time_gpu(chain_bf16, iters, warmup), flops=flops)
    res["chain_fp8qk"] = entry(time_gpu(chain_fp8, iters, warmup), flops=flops)
    res["chain_fp8qk"]["rel_l2_vs_bf16_chain"] = round(float((y8 - y16).norm() / y16.norm()), 4)
    del x, wq, wo, k, v, q8, q8lo, q16, o, cache, y8, y16
    torch.cuda.empty_cache()
    return res


def cpu_baseline(layer):
    """The oracle (fp32 dense-masked CPU path) on the whole FLUX layer with the same masks:
    all active attention rows, GEMM-Q and GEMM-O final over all 36 token blocks; one warm-up pass,
    then timed passes until about 10 s of CPU work (at most 12), median reported."""
    import oracle
    threads = torch.get_num_threads()
    w0, w1, w2 = layer.w0, layer.w1, layer.w2
    cache = torch.zeros(1, 4608, 3072, dtype=torch.bfloat16)

    def one_pass():
        t0 = time.perf_counter()
        oracle.gemm_q(w1.tensors["x"], w1.tensors["w"], 24, w1.packed_info, w1.info_indptr, 0, w1.tensors["bias"])
        t1 = time.perf_counter()
        oracle.sparse_attention(w0.tensors["q"], w0.tensors["k"], w0.tensors["v"], w0.packed_info,
                                w0.packed_kv_info, w0.info_indptr, w0.kv_info_indptr, w0.qo_indptr, w0.kv_indptr)
        t2 = time.perf_counter()
        oracle.gemm_o(w2.tensors["a"], w2.tensors["w"], 24, w2.packed_info, w2.info_indptr, 0, bias=cache,
                      is_for_cache=False)
        t3 = time.perf_counter()
        return t1 - t0, t2 - t1, t3 - t2

    one_pass()
    times, spent = [], 0.0
    while len(times) < 12 and (spent < 10.0 or len(times) < 3):
        t = one_pass()
        times.append(t)
        spent += sum(t)
    med = lambda i: sorted(x[i] for x in times)[len(times) // 2]
    t_q, t_fa, t_o = med(0), med(1), med(2)
    f_q, f_fa, f_o = w1.gemm_q_flops(), w0.attention_flops(), w2.gemm_o_flops(False)
    return {
        "value": round((f_q + f_fa + f_o) / (t_q + t_fa + t_o) / 1e12, 4), "unit": "TFLOP/s", "cores": threads,
        "kind": "port",
        "sample": "whole FLUX layer (GEMM-Q c1, sparse attention c0, GEMM-O final c2), fp32 torch oracle, "
                  "%d timed passes after 1 warm-up, median; %.2f s per pass" % (len(times), t_q + t_fa + t_o),
        "ms_per_step": round((t_q + t_fa + t_o) * 1e3, 2),
        "gemm_q_tflops": round(f_q / t_q / 1e12, 4), "sparse_fa_tflops": round(f_fa / t_fa / 1e12, 4),
        "gemm_o_tflops": round(f_o / t_o / 1e12, 4),
    }


def cpu_baseline_attention(wl, q, k, v, n_random=2048):
    """The oracle on a sample of a big config's attention rows: the first and last q block of every
    head that has them active (short last block, first / last kv range) plus n_random rows drawn with
    a fixed seed.  Reports the measured time and, labelled as an extrapolation, the whole config's time
    = symbol decode (measured in full) + row time scaled by computed kv blocks."""
    import numpy as np
    import oracle
    from oracle.symbols import decode_kv_csr
    s = wl.shape
    n = lambda t: t.numpy()
    t0 = time.perf_counter()
    row_req, row_qb, row_head, ptr, _ = decode_kv_csr(
        n(wl.packed_info), n(wl.packed_kv_info), n(wl.info_indptr), n(wl.kv_info_indptr),
        n(wl.qo_indptr).astype(np.int64), n(wl.kv_indptr).astype(np.int64), s.heads, 128, 128, False)
    t_decode = time.perf_counter() - t0
    n_rows = len(row_req)
    edge = [i for i in range(n_rows) if row_qb[i] in (0, s.n_blocks - 1)]
    rng = np.random.default_rng(5000 + s.index)
    rows = sorted(set(edge) | set(int(i) for i in rng.choice(n_rows, min(n_random, n_rows), replace=False)))
    out = torch.zeros(s.seq, s.heads, 128, dtype=torch.bfloat16)
    call = lambda r: oracle.sparse_attention(q, k, v, wl.packed_info, wl.packed_kv_info, wl.info_indptr,
                                             wl.kv_info_indptr, wl.qo_indptr, wl.kv_indptr, out=out, rows=r)
    call(rows[:8])  # warm-up
    t0 = time.perf_counter()
    call(rows)
    t_rows = time.perf_counter() - t0 - t_decode  # (every call decodes the symbols first)
    blocks = int(sum(int(ptr[i + 1] - ptr[i]) for i in rows))
    total_blocks = int(ptr[n_rows])
    t_full = t_decode + t_rows * total_blocks / blocks
    return {
        "kind": "port", "cores": torch.get_num_threads(),
        "sample": "%d of %d attention rows (%d edge rows: first / last q block; %d random, seeded), %d of %d "
                  "computed kv blocks; symbol decode in full" % (len(rows), n_rows, len(edge), len(rows) - len(edge),
                                                                blocks, total_blocks),
        "measured_s": round(t_rows, 3), "decode_s": round(t_decode, 3),
        "extrapolated_full_s": round(t_full, 2),
        "extrapolated_tflops": round(wl.attention_flops() / t_full / 1e12, 4),
        "extrapolation": "decode_s + measured_s * total kv blocks / sampled kv blocks",
    }


def cpu_baseline_gemms(wl, x, w, bias, n_sample=64):
    """The oracle's GEMM-Q and GEMM-O (final pass) on a sample of a big config's token blocks (the first
    n_sample / 2 and the last n_sample / 2, which includes the short last block); the whole config's time
    is extrapolated by the computed (token block, head) tiles."""
    import oracle
    s = wl.shape
    half = n_sample // 2
    spans = [(0, half * 128), ((s.n_blocks - half) * 128, s.seq)]
    info = wl.sparse_info.to(torch.float64)
    lens = torch.full((s.n_blocks,), 128.0, dtype=torch.float64)
    lens[-1] = s.seq - (s.n_blocks - 1) * 128
    work = (info * lens[:, None]).sum(dim=1)  # active heads x tokens per token block
    sample_work = float(work[:half].sum() + work[s.n_blocks - half:].sum())
    t_q = t_o = 0.0
    for r0, r1 in spans:
        xs = x[:, r0:r1]
        cache = torch.zeros(1, r1 - r0, s.hidden, dtype=torch.bfloat16)
        t0 = time.perf_counter()
        oracle.gemm_q(xs, w, s.heads, wl.packed_info, wl.info_indptr, r0, bias)
        t1 = time.perf_counter()
        oracle.gemm_o(xs, w, s.heads, wl.packed_info, wl.info_indptr, r0, bias=cache, is_for_cache=False)
        t2 = time.perf_counter()
        t_q += t1 - t0
        t_o += t2 - t1
    scale = float(work.sum()) / sample_work
    return {
        "sample": "%d of %d token blocks (first %d, last %d)" % (2 * half, s.n_blocks, half, half),
        "gemm_q_measured_s": round(t_q, 3), "gemm_o_final_measured_s": round(t_o, 3),
        "gemm_q_extrapolated_full_s": round(t_q * scale, 2), "gemm_o_final_extrapolated_full_s": round(t_o * scale, 2),
        "gemm_q_extrapolated_tflops": round(wl.gemm_q_flops() / (t_q * scale) / 1e12, 4),
        "gemm_o_final_extrapolated_tflops": round(wl.gemm_o_flops(False) / (t_o * scale) / 1e12, 4),
        "extrapolation": "measured_s * active (token block, head) tiles of the config / of the sample",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=300,
                    help="untimed steps; the clocks of an idle device need ~100 ms of load to settle")
    ap.add_argument("--configs", default="0,1,2,3,4")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="skip the captured-graph replay of the step")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB elementwise copy kernel (known FETCH/WRITE size) so "
                         "that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path runs on a single MI355X (heads shard without "
                 "communication; nothing here uses a second GPU). Run with --gpus 1.")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    configs = {int(c) for c in args.configs.split(",") if c != ""}
    K, W = args.steps, args.warmup

    if args.copy_calibration:
        src = torch.ones(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(4):
            torch.bitwise_not(src, out=dst)  # one kernel that reads 256 MiB and writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
    log("[bench] building FLUX layer inputs (configs 0-2)")
    layer = FluxLayer(dev)
    kernels = {}

    # the step's two-stream form must give what the plain sequence of calls gives
    layer.gemm_q(); layer.attention(fresh_decode=True); ref_o = layer.gemm_o_final().clone()
    ref_q, ref_fa = layer.out_q.clone(), layer.out_fa.clone()
    layer.out_q.zero_(); layer.out_fa.zero_()
    got_o = layer.step()
    torch.cuda.synchronize()
    assert torch.equal(ref_q, layer.out_q) and torch.equal(ref_fa, layer.out_fa) and torch.equal(ref_o, got_o), \
        "two-stream step differs from the sequential chain"
    del ref_q, ref_fa, ref_o, got_o

    # ---- clock settle (fixed, whatever --warmup says), W warm-up steps, then the timed region ----
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < SETTLE_MS:
        for _ in range(20):
            layer.step()
        torch.cuda.synchronize()
    settle_ms = (time.perf_counter() - t_settle) * 1e3
    for _ in range(W):
        layer.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        layer.step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / K
    chain_flops = layer.chain_flops()
    value = chain_flops / (ms_per_step * 1e-3) / 1e12
    log("[bench] chain %.4f ms/step -> %.1f TFLOP/s" % (ms_per_step, value))

    # ---- the reference's call sequence on one stream (the decode inside run(), nothing overlapped) ----
    for _ in range(W):
        layer.step_dropin()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        layer.step_dropin()
    torch.cuda.synchronize()
    dropin_ms = (time.perf_counter() - t0) * 1e3 / K
    log("[bench] drop-in call sequence %.4f ms/step -> %.1f TFLOP/s" % (dropin_ms, chain_flops / (dropin_ms * 1e-3) / 1e12))

    # ---- the same step as one captured HIP graph (the reference declares run() capturable,
    # flashomni/attention.py:140-141): reported beside the eager figure, which stays `value` ----
    graph_ms, graph_error = None, None
    if not args.no_graph:
        try:
            graph_ms = captured_step_ms(layer, dev, K, W)
            log("[bench] captured step %.4f ms/replay -> %.1f TFLOP/s" % (graph_ms, chain_flops / (graph_ms * 1e-3) / 1e12))
        except Exception as e:  # (reported in the line; the eager figures do not depend on this leg)
            graph_error = "%s: %s" % (type(e).__name__, e)
            log("[bench] captured step failed: " + graph_error)

    # ---- per-kernel, HIP events ----
    # (these launches last 0.02-0.15 ms: whatever --steps / --warmup say, each is timed over at least
    # 100 launches after at least 100 untimed ones, so that a short run does not time them at clocks
    # that are still moving)
    KK, WW = max(K, 100), max(W, 100)
    w0 = layer.w0
    c0 = {}
    # (the attention launch first, straight after the step loop: the decoder's 17 us launches in between
    # would let the clocks fall back)
    fa_ms = time_gpu(lambda: layer.attention(fresh_decode=False), KK, WW)
    ms = time_gpu(layer.decode, KK, WW)
    rows, nnz = layer.wrapper._worklist.sizes()
    c0["decode"] = entry(ms, nbytes=w0.packed_info.numel() + w0.packed_kv_info.numel() + 4 * (4 * rows + 1 + nnz))
    c0["decode"]["rows"], c0["decode"]["kv_blocks"] = rows, nnz
    c0["sparse_fa_bf16"] = entry(fa_ms, flops=w0.attention_flops())
    c0["sparse_fa_bf16"]["computed_blocks"] = w0.computed_blocks
    # the call a user of the reference makes: decode of the symbols + attention, every time
    c0["run_dropin"] = entry(time_gpu(lambda: layer.attention(fresh_decode=True), KK, WW), flops=w0.attention_flops())
    kernels[w0.shape.name] = c0
    ms = time_gpu(layer.gemm_q, KK, WW)
    kernels[layer.w1.shape.name] = {"gemm_q": entry(ms, flops=layer.w1.gemm_q_flops())}
    kernels[layer.w1.shape.name]["gemm_q"]["tiles"] = layer.w1.active_rows
    c2 = {}
    c2["gemm_o_cache"] = entry(time_gpu(layer.gemm_o_cache, KK, WW), flops=layer.w2.gemm_o_flops(True))
    c2["gemm_o_final"] = entry(time_gpu(layer.gemm_o_final, KK, WW), flops=layer.w2.gemm_o_flops(False))
    kernels[layer.w2.shape.name] = c2
    # packbits at the config-0 mask size, at 16 Mi flags (both bounded by the host's call rate: the
    # kernel is shorter than a call) and at 256 Mi flags (bounded by HBM)
    pk = {}
    for n in (31104, 1 << 24, 1 << 28):
        xb = (torch.rand(n, device=dev) < 0.5)
        pk["n=%d" % n] = entry(time_gpu(lambda: layer.fo.packbits(xb, "little"), K, W), nbytes=n + n // 8)
    kernels["packbits"] = pk
    # symbol producer (pooled scores -> packed symbols) at the block grids of configs 0, 3 and 4
    from flashomni_amd.workloads import SHAPES
    sp = {}
    for idx in (0, 3, 4):
        if idx not in configs:
            continue
        sh = SHAPES[idx]
        gen = torch.Generator(device=dev).manual_seed(2000 + idx)
        pooled = torch.randn(1, sh.heads, sh.n_blocks, sh.n_blocks, generator=gen, device=dev) * 2.0
        thr = torch.full((sh.heads,), 0.3, device=dev)
        it, wm = (K, W) if idx == 0 else (max(3, min(K, 20)), 3)
        ms = time_gpu(lambda: layer.fo.sparse_symbols_from_scores(pooled, 4, 0.2, thr), it, wm)
        sp[sh.name] = entry(ms, nbytes=pooled.numel() * 4 + pooled.numel() // 8)
        sp[sh.name]["rows"] = sh.heads * sh.n_blocks
        del pooled
    kernels["symbols_from_scores"] = sp
    for name, d in kernels.items():
        log("[bench]", name, json.dumps(d))

    # (the millisecond-scale launches of configs 3 and 4: a few tens of milliseconds of the same launch before
    # timing, so that clocks and caches are those of a steady run)
    big_iters, big_warm = max(3, min(K, 20)), 8
    cpu_big = {}
    for idx in (3, 4):
        if idx in configs:
            log("[bench] config %d attention (bf16)" % idx)
            res, cpu_fa = bench_big_attention(dev, idx, big_iters, big_warm, with_cpu=not args.no_cpu)
            if cpu_fa is not None:
                cpu_big["c%d" % idx] = {"sparse_fa": cpu_fa}
            if idx == 4:
                log("[bench] config 4 GEMMs + quantiser")
                res_g, cpu_g = bench_big_gemms(dev, idx, big_iters, big_warm, with_cpu=not args.no_cpu)
                res.update(res_g)
                if cpu_g is not None:
                    cpu_big["c4"]["gemms"] = cpu_g
                log("[bench] config 4 chain end to end")
                res.update(bench_wan_chain(dev, big_iters, big_warm))
            kernels[SHAPES[idx].name] = res
            log("[bench]", SHAPES[idx].name, json.dumps(res))

    # what the step costs beyond its three kernels (the decode runs beside GEMM-Q on a second stream)
    kernel_sum_ms = (kernels[layer.w1.shape.name]["gemm_q"]["ms"] + fa_ms
                     + kernels[layer.w2.shape.name]["gemm_o_final"]["ms"])
    fa_flops = w0.attention_flops()
    traffic, traffic_state = traffic_from_profile()
    roofline = {
        "kernel": "sparse_fa_kernel<bf16> (config 0, FLUX shape)", "bound": "mfma",
        "achieved": round(fa_flops / (fa_ms * 1e-3) / 1e12, 2), "peak": PEAK_BF16, "unit": "TFLOP/s",
        "frac": round(fa_flops / (fa_ms * 1e-3) / 1e12 / PEAK_BF16, 4),
        # HBM bytes per launch: read from the committed summary of two rocprofv3 --pmc runs of this
        # command (FETCH_SIZE and WRITE_SIZE, each scaled by what a 256 MiB copy kernel reads on the same
        # counter); the algorithmic bytes of the launch are 98.6e6
        "traffic": traffic, "traffic_state": traffic_state, "traffic_unit": "bytes/launch",
        "traffic_source": "profiles/" + os.path.basename(TRAFFIC_PROFILE),
        "launch_ms": round(fa_ms, 5), "algorithmic_flop_per_launch": fa_flops,
    }
    cpu = None
    if not args.no_cpu:
        log("[bench] CPU baseline (oracle, %d threads)" % torch.get_num_threads())
        cpu = cpu_baseline(layer)
        cpu.update(cpu_big)

    line = {
        "metric": "sparse-FA + GEMM-Q/O effective TFLOP/s on computed blocks, FLUX-shaped sparse layer "
                  "(GEMM-Q c1 -> decode + sparse FA c0 -> GEMM-O final c2), 1 GPU",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 5), "settle_ms": round(settle_ms, 1),
        "host_gap_ms": round(ms_per_step - kernel_sum_ms, 5),
        "dropin_call_sequence": {
            "ms_per_step": round(dropin_ms, 5), "tflops": round(chain_flops / (dropin_ms * 1e-3) / 1e12, 2),
            "note": "flashomni_gemm -> wrapper.run(q, k, v, symbols) -> flashomni_gemm_reduction on one stream, "
                    "the decode inside run(); `value` overlaps the decode with GEMM-Q on a second stream"},
        "captured_graph": {"error": graph_error} if graph_ms is None else {
            "ms_per_step": round(graph_ms, 5), "tflops": round(chain_flops / (graph_ms * 1e-3) / 1e12, 2),
            "note": "the same two-stream step replayed as one HIP graph; `value` is the eager step"},
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "FLUX layer: c1_flux_gemm_q + c0_flux_sparse_fa + c2_flux_gemm_o(final)",
                   "seq": 4608, "heads": 24, "head_dim": 128, "hidden": 3072, "block": 128,
                   "p_cached": 0.25, "kv_density": round(float(w0.sparse_kv_info.float().mean()), 3),
                   "frac_of_bf16_peak": round(value / PEAK_BF16, 4)},
        "roofline": roofline, "cpu_baseline": cpu, "kernels": kernels,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
