"""CPU: the C-ABI library loads and exports every declared symbol; the host planner
(fo_prefill_plan, fo_sparse_block_table, fo_decode_sizes) agrees with the oracle planner and with
closed forms; workload generators hit the stated mask densities."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import oracle
from oracle.planner import binary_search_kv_chunk, determine_cta_tile_q

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib():
    from flashomni_amd import _lib
    return _lib


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "flashomni_hip.h")).read()
    declared = set(re.findall(r"\b(fo_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 12
    L = _lib()
    handle = ctypes.CDLL(L.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), name
    assert declared == set(L.SIGNATURES), declared ^ set(L.SIGNATURES)
    assert L.lib().fo_abi_version() == int(re.search(r"#define\s+FO_ABI_VERSION\s+(\d+)", header).group(1)) == 5


_C_SCALARS = {"int": ctypes.c_int, "int32_t": ctypes.c_int32, "uint32_t": ctypes.c_uint32,
              "int64_t": ctypes.c_int64, "uint64_t": ctypes.c_uint64, "size_t": ctypes.c_size_t,
              "float": ctypes.c_float, "double": ctypes.c_double}


def test_ctypes_signatures_follow_the_header():
    """Every parameter the header declares has a ctypes argument of the same kind and width in the
    same position (a pointer or array -> a pointer-sized argument), and the return types agree: a
    changed entry point cannot drift from its binding unnoticed."""
    header = open(os.path.join(ROOT, "include", "flashomni_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    header = re.sub(r"//[^\n]*", "", header)
    L = _lib()
    seen = 0
    for m in re.finditer(r"([A-Za-z_][A-Za-z0-9_ ]*?[\s\*]+)(fo_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", header):
        ret, name, args = m.group(1).strip(), m.group(2), m.group(3).strip()
        params = [] if args in ("", "void") else [a.strip() for a in args.split(",")]
        argtypes, restype = L.SIGNATURES[name]
        assert len(params) == len(argtypes), name
        for i, (decl, ct) in enumerate(zip(params, argtypes)):
            if "*" in decl or "[" in decl:
                assert ctypes.sizeof(ct) == ctypes.sizeof(ctypes.c_void_p) and ct in (
                    ctypes.c_void_p, ctypes.c_char_p), (name, i, decl)
                continue
            words = [w for w in decl.split() if w not in ("const", "unsigned", "signed")]
            want = _C_SCALARS[words[-2]]
            assert ctypes.sizeof(ct) == ctypes.sizeof(want), (name, i, decl)
            assert (ct in (ctypes.c_float, ctypes.c_double)) == (want in (ctypes.c_float, ctypes.c_double)), \
                (name, i, decl)
        ret_words = [w for w in ret.replace("*", " * ").split() if w not in ("const", "extern", "FO_API")]
        if "*" in ret_words:
            assert restype in (ctypes.c_char_p, ctypes.c_void_p), name
        elif ret_words[-1] == "void":
            assert restype is None, name
        else:
            assert ctypes.sizeof(restype) == ctypes.sizeof(_C_SCALARS[ret_words[-1]]), name
        seen += 1
    assert seen == len(L.SIGNATURES)


def _plan(qo, kv, hq, hkv, d, num_cu=256, int_ws=8 << 20, float_ws=128 << 20, graph=False, total=None):
    L = _lib()
    qo_t, kv_t = torch.tensor(qo, dtype=torch.int32), torch.tensor(kv, dtype=torch.int32)
    host = torch.zeros(int_ws, dtype=torch.uint8)
    info = torch.zeros(15, dtype=torch.int64)
    rc = L.lib().fo_prefill_plan(None, float_ws, None, host.data_ptr(), int_ws, qo_t.data_ptr(),
                                 kv_t.data_ptr(), total if total is not None else qo[-1], len(qo) - 1,
                                 hq, hkv, d, d, 1, int(graph), 2, num_cu, info.data_ptr(), None)
    return rc, info.tolist(), host


CASES = [
    ([0, 4608], [0, 4608], 24),                    # FLUX: 36 tiles, no split
    ([0, 33280], [0, 33280], 24),
    ([0, 76112], [0, 76112], 40),
    ([0, 300, 301, 429, 1429], [0, 77, 590, 718, 4814], 3),   # ragged: kv split kicks in
    ([0, 16], [0, 100000], 8),                     # short q, long kv
    ([0, 40, 80], [0, 5000, 10000], 2),
]


@pytest.mark.parametrize("qo,kv,heads", CASES)
def test_planner_matches_oracle(qo, kv, heads):
    rc, info, host = _plan(qo, kv, heads, heads, 128)
    assert rc == 0, _lib().lib().fo_last_error()
    exp = oracle.prefill_plan(qo, kv, heads, heads, 128, 256)
    assert info == exp["plan_info"]
    arr = lambda off, n: host[off:off + 4 * n].view(torch.int32).tolist()
    n = exp["padded_batch_size"]
    assert arr(info[4], n) == exp["request_indices"]
    assert arr(info[5], n) == exp["qo_tile_indices"]
    assert arr(info[6], n) == exp["kv_tile_indices"]
    assert arr(info[8], len(qo)) == exp["o_indptr"]
    assert arr(info[9], 1) == [exp["kv_chunk_size"]]
    if exp["split_kv"]:
        assert arr(info[7], qo[-1] + 1) == exp["merge_indptr"]
        assert host[info[12]:info[12] + n].tolist() == [1] * n


def test_planner_closed_forms_at_the_benchmark_shapes():
    for seq, heads, tiles in ((4608, 24, 36), (33280, 24, 260), (76112, 40, 595)):
        rc, info, _ = _plan([0, seq], [0, seq], heads, heads, 128)
        assert rc == 0
        assert info[0] == tiles and info[3] == 128 and info[14] == 0     # padded batch, tile q, no split
    assert determine_cta_tile_q(65, 128) == 128 and determine_cta_tile_q(64, 128) == 64
    assert determine_cta_tile_q(16, 128) == 16 and determine_cta_tile_q(1000, 256) == 64


def test_kv_chunk_binary_search_is_minimal():
    for packed, kvl, limit in (([16], [100000], 64), ([300, 40], [5000, 9000], 21), ([128], [128], 10)):
        split, chunk = binary_search_kv_chunk(False, limit, packed, kvl, 16, 128)
        tiles = lambda c: sum(-(-q // 16) * -(-max(k, 1) // c) for q, k in zip(packed, kvl))
        hi = max(kvl)
        if tiles(hi) > limit:        # even unsplit kv does not fit: the search saturates at max kv
            assert chunk == hi
        elif chunk > 128:
            assert tiles(chunk) <= limit < tiles(chunk - 1)
        assert split == (chunk < hi)


def test_planner_errors():
    L = _lib().lib()
    rc, _, _ = _plan([0, 128], [0, 128], 3, 2, 128)
    assert rc < 0 and b"divisible" in L.fo_last_error()
    rc, _, _ = _plan([0, 128, 64], [0, 128, 256], 2, 2, 128)
    assert rc < 0 and b"non-negative" in L.fo_last_error()
    rc, _, _ = _plan([0, 4608], [0, 4608], 24, 24, 128, int_ws=64)
    assert rc == -2 and b"integer workspace" in L.fo_last_error()
    rc, _, _ = _plan([0, 16], [0, 100000], 8, 8, 128, float_ws=1024)
    assert rc == -2 and b"float workspace" in L.fo_last_error()


def test_block_table_and_decode_sizes():
    L = _lib().lib()
    qo = torch.tensor([0, 300, 301, 429], dtype=torch.int32)
    kv = torch.tensor([0, 77, 590, 718], dtype=torch.int32)
    out = torch.zeros(3, dtype=torch.int64)
    assert L.fo_decode_sizes(qo.data_ptr(), kv.data_ptr(), 3, 5, 128, 128, out[0:].data_ptr(),
                             out[1:].data_ptr(), out[2:].data_ptr()) == 0
    assert out.tolist() == [5, 25, (3 * 1 + 1 * 5 + 1 * 1) * 5]
    table = torch.zeros(2, 5, dtype=torch.int32)
    n = torch.zeros(1, dtype=torch.int64)
    assert L.fo_sparse_block_table(qo.data_ptr(), 3, 128, table[0].data_ptr(), table[1].data_ptr(), 5,
                                   n.data_ptr()) == 0
    assert table.tolist() == [[0, 0, 0, 1, 2], [0, 1, 2, 0, 0]] and int(n) == 5
    assert L.fo_sparse_block_table(qo.data_ptr(), 3, 128, table[0].data_ptr(), table[1].data_ptr(), 4,
                                   n.data_ptr()) == -2


def test_argument_checks_without_gpu():
    """Entry points validate before touching the device."""
    L = _lib().lib()
    assert L.fo_packbits(None, 8, 7, None, None) == -1 and b"bitorder" in L.fo_last_error()
    assert L.fo_gemm_q(1, 1, None, 1, 0, 1, 128, 100, 64, 128, 1, None, None, 0, 1, None, 0, None) == -1
    assert b"only support" in L.fo_last_error()
    assert L.fo_sparse_fa_run(*([None] * 5), 0, None, None, None, None, *([0] * 8), *([None] * 4), 0, 0, *([None] * 7), 4, 2, 2, 0, 64, 128, 128,
                              1.0, 0.0, None, None, 0, None) == -1
    assert b"head_dim" in L.fo_last_error()
    # the logits soft cap: finite, >= 0, 16-bit q/k only
    tail = (None, None, 0, None)
    head = (*([None] * 5),)
    mid = (None, None, None, None, *([0] * 8), *([None] * 4), 0, 0, *([None] * 7), 4, 2, 2, 0, 128, 128, 128, 1.0)
    assert L.fo_sparse_fa_run(*head, 0, *mid, -1.0, *tail) == -1 and b"logits_soft_cap" in L.fo_last_error()
    assert L.fo_sparse_fa_run(*head, 0, *mid, float("inf"), *tail) == -1 and b"logits_soft_cap" in L.fo_last_error()
    assert L.fo_sparse_fa_run(*head, 2, *mid, 30.0, *tail) == -1 and b"soft cap" in L.fo_last_error()


def test_ops_fail_loudly_without_a_gpu_or_library(monkeypatch):
    import flashomni_amd as fo
    with pytest.raises(ValueError, match="GPU"):
        fo.packbits(torch.ones(8, dtype=torch.bool))
    with pytest.raises(ValueError, match="GPU"):
        fo.flashomni_gemm(torch.zeros(1, 128, 64, dtype=torch.bfloat16),
                          torch.zeros(128, 64, dtype=torch.bfloat16), 1, is_full=True)
    with pytest.raises(ValueError, match="GPU"):
        fo.BatchFlashOmniFAWithRaggedKVWrapper(torch.empty(16, dtype=torch.uint8))
    L = _lib()
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", "/nonexistent/libflashomni_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        L.lib()


def test_workload_mask_densities():
    from flashomni_amd.workloads import make_workload
    w0 = make_workload(0, tensors=False)
    assert w0.sparse_info.shape == (36, 24) and w0.sparse_kv_info.shape == (36, 24, 36)
    assert 0.70 < w0.sparse_info.float().mean() < 0.80
    assert 0.54 < w0.sparse_kv_info.float().mean() < 0.60
    assert bool(w0.sparse_kv_info[:, :, :4].all())
    assert bool(w0.sparse_kv_info[torch.arange(36), :, torch.arange(36)].all())
    assert w0.packed_info.numel() == 108 and w0.packed_kv_info.numel() == 3888
    w1 = make_workload(1, tensors=False)
    assert torch.equal(w1.sparse_info, w0.sparse_info)        # configs 1/2 reuse config 0's flags
    w3 = make_workload(3, tensors=False)
    assert 0.18 < w3.sparse_kv_info.float().mean() < 0.24
