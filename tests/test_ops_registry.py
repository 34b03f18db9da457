"""CPU: the six ``torch.ops.flashomni_kernels`` operators exist with the reference's signatures.

The expected lists restate the C++ declarations of csrc/flashomni_ops.cu:20-51 (argument order and
kinds) so that the check does not need the reference tree at run time."""
import pytest
import torch

import flashomni_amd  # noqa: F401  (registers the operators)
from flashomni_amd import attention as fa_attention

T, TO, I, B, F, S = "Tensor", "Tensor?", "int", "bool", "float", "str"
EXPECTED = {
    # at::Tensor BatchSparseFAWithKVPlan(...)  csrc/flashomni_ops.cu:20-25
    "batch_sparseFA_with_kv_plan": ([T, T, T, T, T, T, I, I, I, I, I, B, I, I], "Tensor"),
    # void BatchSparseFAWithRaggedKVRun(...)  :27-35 + the seven additional parameters of
    # aot_build_utils/generate_aot_default_additional_params_header.py:78-89
    "batch_sparseFA_with_ragged_kv_run": ([T, T, T, T, T, T, TO, TO, TO, TO, I, I, B, T, T, T, TO, I, I,
                                           TO, TO, TO, F, F, F, F], "()"),
    # void FLASHOMNIGEMM(...)  :38-39
    "flashomni_gemm": ([T, T, T, TO, I, I, TO, TO, I, B], "()"),
    # void FLASHOMNIGEMMReduction(...)  :42-43
    "flashomni_gemm_reduction": ([T, T, T, TO, I, I, T, T, I, B], "()"),
    # void packbits(at::Tensor x, const std::string& bitorder, at::Tensor y)  :48
    "packbits": ([T, S, T], "()"),
    # void segment_packbits(x, input_indptr, output_indptr, bitorder, y)  :50-51
    "segment_packbits": ([T, T, T, S, T], "()"),
}


def _kind(arg):
    s = str(arg.type)
    return {"Optional[Tensor]": TO}.get(s, s)


@pytest.mark.parametrize("name", sorted(EXPECTED))
def test_operator_registered_with_reference_signature(name):
    op = getattr(torch.ops.flashomni_kernels, name).default
    kinds, ret = EXPECTED[name]
    got = [_kind(a) for a in op._schema.arguments]
    assert got == kinds
    rets = op._schema.returns
    assert (ret == "()" and len(rets) == 0) or (ret == "Tensor" and len(rets) == 1 and str(rets[0].type) == "Tensor")
    assert all(a.default_value is None and not a.kwarg_only for a in op._schema.arguments)  # all positional


def test_exactly_the_reference_names():
    assert set(flashomni_amd.ops.OP_NAMES) == set(EXPECTED)


def test_operators_have_no_cpu_path():
    x = torch.ones(8, dtype=torch.bool)
    y = torch.zeros(1, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="GPU"):
        torch.ops.flashomni_kernels.packbits.default(x, "big", y)
    with pytest.raises(RuntimeError, match="bitorder must be 'big' or 'little'"):
        torch.ops.flashomni_kernels.packbits.default(x, "middle", y)


def test_bit_count_indptr_helpers_closed_form():
    """flashomni/attention.py:165-191: cumsum(ceil(qo/bs)*H) and cumsum(ceil(qo/bs)*ceil(kv/bs)*H);
    config 0 (one request of 4608 tokens, 24 heads) gives [0, 864] and [0, 31104]."""
    qo = torch.tensor([0, 4608], dtype=torch.int32)
    a = fa_attention._compute_sparse_info_indptr(qo, 24, 128, device="cpu")
    b = fa_attention._compute_sparse_kv_info_indptr(qo, qo, 24, 128, 128, device="cpu")
    assert a.tolist() == [0, 864] and b.tolist() == [0, 31104]
    qo = torch.tensor([0, 300, 301, 1000], dtype=torch.int32)
    kv = torch.tensor([0, 77, 590, 718], dtype=torch.int32)
    a = fa_attention._compute_sparse_info_indptr(qo, 3, 128, device="cpu")
    b = fa_attention._compute_sparse_kv_info_indptr(qo, kv, 3, 128, 128, device="cpu")
    assert a.tolist() == [0, 9, 12, 30]                   # 3, 1, 6 q blocks x 3 heads
    assert b.tolist() == [0, 9, 9 + 3 * 5, 9 + 15 + 18]   # x 1, 5, 1 kv blocks
