"""GPU parity of the 14B-video layer chain (config 4) at full size: GEMM-Q -> [fp8 quantisation of Q
and K] -> block-sparse attention -> GEMM-O final pass, seq 76 112 (80-row last block), 40 heads,
hidden 5120, against the oracle chain evaluated on sampled token blocks.

The oracle chain is the fp32 dense masked CPU path with the reference's intermediate dtypes (Q and
the attention output are bf16 tensors between the operators) and no quantisation anywhere.
Tolerances: bf16 chain max-abs 2e-2 and relative L2 1e-2; fp8 chain relative L2 3e-2."""
import math

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

N_RANDOM_BLOCKS = 8


class _Chain:
    """Inputs of the chain on the GPU, its two GPU results, and the oracle on sampled token blocks."""

    def __init__(self, dev):
        import flashomni_amd as fo
        from flashomni_amd.workloads import make_workload
        self.fo, self.dev = fo, dev
        wl = self.wl = make_workload(4, tensors=False)
        s = self.s = wl.shape
        M, C, H = s.seq, s.hidden, s.heads
        g = torch.Generator(device=dev).manual_seed(4004)
        rnd = lambda *sz, std=1.0: (torch.randn(*sz, generator=g, device=dev) * std).to(torch.bfloat16)
        self.x, self.wq, self.bq = rnd(1, M, C), rnd(C, C, std=0.02), rnd(C, std=0.02)
        self.wo = rnd(C, C, std=0.02)
        self.k, self.v = rnd(M, H, 128), rnd(M, H, 128)
        # the attention output of the previous step, whose cached heads the final GEMM-O pass reuses
        self.o_prev = rnd(M, H, 128, std=0.05)
        self.sym = [t.to(dev) for t in (wl.packed_info, wl.packed_kv_info, wl.info_indptr, wl.kv_info_indptr)]
        self.ws = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        self.cache = fo.flashomni_gemm_reduction(self.o_prev.view(1, M, C), self.wo, H, self.sym[0], self.sym[2],
                                                 0, bias=None, is_for_cache=True)

    def run_bf16(self):
        fo, s = self.fo, self.s
        M, C, H = s.seq, s.hidden, s.heads
        q16 = torch.zeros(1, M, C, dtype=torch.bfloat16, device=self.dev)
        fo.flashomni_gemm(self.x, self.wq, H, self.sym[0], self.sym[2], 0, self.bq, out=q16)
        w = fo.BatchFlashOmniFAWithRaggedKVWrapper(self.ws)
        w.plan(self.wl.qo_indptr, self.wl.kv_indptr, H, H, 128, q_data_type=torch.bfloat16)
        o = self.o_prev.clone()
        w.run(q16.view(M, H, 128), self.k, self.v, self.sym[0], self.sym[1], self.sym[2], self.sym[3], out=o)
        y = fo.flashomni_gemm_reduction(o.view(1, M, C), self.wo, H, self.sym[0], self.sym[2], 0, bias=self.cache,
                                        is_for_cache=False)
        return o, y

    def run_fp8(self, two_term=True, two_term_k=False):
        fo, s = self.fo, self.s
        M, C, H = s.seq, s.hidden, s.heads
        res = fo.flashomni_gemm(self.x, self.wq, H, self.sym[0], self.sym[2], 0, self.bq, out=False,
                                quant_out="residual" if two_term else True)
        q8, qs = res[1], res[2]
        q_lo = res[3].view(M, H, 128) if two_term else None
        k8, ks, k_lo = fo.quant_fp8_block(self.k, self.wl.kv_indptr, residual=True)
        if not two_term_k:
            k_lo = None
        w = fo.BatchFlashOmniFAWithRaggedKVWrapper(self.ws)
        w.plan(self.wl.qo_indptr, self.wl.kv_indptr, H, H, 128, q_data_type=torch.float8_e4m3fn)
        o = self.o_prev.clone()
        w.run(q8.view(M, H, 128), k8, self.v, self.sym[0], self.sym[1], self.sym[2], self.sym[3], out=o,
              q_scale=qs, k_scale=ks, q_lo=q_lo, k_lo=k_lo)
        y = fo.flashomni_gemm_reduction(o.view(1, M, C), self.wo, H, self.sym[0], self.sym[2], 0, bias=self.cache,
                                        is_for_cache=False)
        return o, y

    def oracle_blocks(self):
        """[(r0, r1, attention output [rows, H, 128] bf16, chain output [rows, C] bf16)] for the first
        and the short last token block plus seeded random ones."""
        wl, s = self.wl, self.s
        M, C, H = s.seq, s.hidden, s.heads
        rng = np.random.default_rng(44)
        blocks = sorted({0, s.n_blocks - 1, *rng.choice(s.n_blocks, N_RANDOM_BLOCKS, replace=False).tolist()})
        _, row_qb, _, _, _ = oracle.decode_kv_csr(
            wl.packed_info.numpy(), wl.packed_kv_info.numpy(), wl.info_indptr.numpy(), wl.kv_info_indptr.numpy(),
            wl.qo_indptr.numpy(), wl.kv_indptr.numpy(), H, 128, 128)
        k_c, v_c = self.k.cpu(), self.v.cpu()
        wq_c, bq_c, wo_c = self.wq.cpu(), self.bq.cpu(), self.wo.cpu()
        q_c = torch.zeros(M, H, 128, dtype=torch.bfloat16)
        o_c = self.o_prev.cpu()
        o_prev_c = o_c.clone()
        out = []
        for b in blocks:
            r0, r1 = b * 128, min(M, b * 128 + 128)
            q_blk = oracle.gemm_q(self.x[:, r0:r1].cpu(), wq_c, H, wl.packed_info, wl.info_indptr, r0, bq_c,
                                  out=torch.zeros(1, r1 - r0, C, dtype=torch.bfloat16))
            q_c[r0:r1] = q_blk.view(r1 - r0, H, 128)
            rows = [int(i) for i in np.nonzero(row_qb == b)[0]]
            oracle.sparse_attention(q_c, k_c, v_c, wl.packed_info, wl.packed_kv_info, wl.info_indptr,
                                    wl.kv_info_indptr, wl.qo_indptr, wl.kv_indptr, out=o_c, rows=rows)
            cache = oracle.gemm_o(o_prev_c[r0:r1].reshape(1, r1 - r0, C), wo_c, H, wl.packed_info, wl.info_indptr,
                                  r0, bias=None, is_for_cache=True)
            y = oracle.gemm_o(o_c[r0:r1].reshape(1, r1 - r0, C), wo_c, H, wl.packed_info, wl.info_indptr, r0,
                              bias=cache, is_for_cache=False)
            out.append((r0, r1, o_c[r0:r1].clone(), y[0]))
        return out


@pytest.fixture(scope="module")
def chain(dev):
    c = _Chain(dev)
    c.expected = c.oracle_blocks()
    yield c
    del c
    torch.cuda.empty_cache()


def _errors(got_o, got_y, expected, C):
    """max-abs and relative L2 over the sampled blocks, for the attention output and the chain output."""
    acc = {"o": [0.0, 0.0, 0.0], "y": [0.0, 0.0, 0.0]}
    for r0, r1, exp_o, exp_y in expected:
        for name, got, exp in (("o", got_o[r0:r1].cpu(), exp_o), ("y", got_y[0, r0:r1].cpu(), exp_y)):
            d = got.float() - exp.float()
            acc[name][0] = max(acc[name][0], float(d.abs().max()))
            acc[name][1] += float((d ** 2).sum())
            acc[name][2] += float((exp.float() ** 2).sum())
    return {n: (a[0], math.sqrt(a[1] / a[2])) for n, a in acc.items()}


def test_chain_bf16(chain):
    o, y = chain.run_bf16()
    err = _errors(o, y, chain.expected, chain.s.hidden)
    print("bf16 chain: attention max-abs %.4g rel-L2 %.4g; output max-abs %.4g rel-L2 %.4g" % (*err["o"], *err["y"]))
    assert err["o"][0] <= 2e-2 and err["o"][1] <= 1e-2
    assert err["y"][0] <= 2e-2 and err["y"][1] <= 1e-2
    # the short last block is among the sampled ones, and cached strips kept the previous step's bytes
    assert chain.expected[-1][1] - chain.expected[-1][0] == 80
    active = chain.wl.sparse_info.to(chain.dev).repeat_interleave(128, dim=0)[:chain.s.seq]
    assert torch.equal(o[~active].view(torch.int16), chain.o_prev[~active].view(torch.int16))


def test_chain_fp8_contract(chain):
    """The stated fp8 tolerance on the chain's own data: relative L2 3e-2 against the unquantised oracle.
    e4m3 keeps 3 mantissa bits: rounding k alone puts noise of 0.026 x rms(q) x rms(k) on every logit, and
    this chain's q = x . W_q^T (W_q ~ N(0, 0.02), hidden 5120) has rms 1.43, so a k stored in one e4m3 byte
    cannot meet 3e-2 whatever is done with q (test_chain_fp8_error_level).  The chain therefore runs q and k
    in two e4m3 terms each (value + rounding residual under one scale per (head, block))."""
    o, y = chain.run_fp8(two_term=True, two_term_k=True)
    err = _errors(o, y, chain.expected, chain.s.hidden)
    print("fp8 chain, two-term q and k: attention max-abs %.4g rel-L2 %.4g; output max-abs %.4g rel-L2 %.4g"
          % (*err["o"], *err["y"]))
    assert err["o"][1] <= 3e-2 and err["y"][1] <= 3e-2


def test_chain_fp8_error_level(chain):
    """Not the contract (see test_chain_fp8_contract): pins the error of the chain with k in ONE e4m3 term
    to the level the rounding of k explains, so that a kernel defect on that path still shows.  With q in
    one e4m3 term as well the error is sqrt(2) times larger."""
    o2, y2 = chain.run_fp8(two_term=True)
    e2 = _errors(o2, y2, chain.expected, chain.s.hidden)
    o1, y1 = chain.run_fp8(two_term=False)
    e1 = _errors(o1, y1, chain.expected, chain.s.hidden)
    print("fp8 chain, two-term q: attention rel-L2 %.4g, output rel-L2 %.4g; one-term q: %.4g, %.4g"
          % (e2["o"][1], e2["y"][1], e1["o"][1], e1["y"][1]))
    assert e2["o"][1] <= 4.5e-2 and e2["y"][1] <= 4.5e-2
    assert e1["o"][1] <= 6.5e-2 and e1["y"][1] <= 6.5e-2
    assert e2["y"][1] < 0.8 * e1["y"][1]
