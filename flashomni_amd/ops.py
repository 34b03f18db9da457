"""``torch.ops.flashomni_kernels``: the reference's six native operators over the C ABI.

The reference's Python modules reach their kernels through
``torch.ops.flashomni_kernels.<name>.default`` (flashomni/attention.py:59-65,
flashomni/gemm.py:41-43, flashomni/quantization.py:31-34); the operators are registered by
csrc/flashomni_ops.cu:55-68 with the C++ signatures of :20-51.  Importing this module registers the
same six names with the same positional signatures, so the reference's own ``flashomni/*.py`` runs
unchanged on top of this library.

The attention pair needs state the reference's signatures have no slot for (the decoder's q-block
table and the work-list buffers).  ``batch_sparseFA_with_kv_plan`` builds it and files it under the
address of the integer workspace it was given; ``batch_sparseFA_with_ragged_kv_run`` finds it there,
as the reference's run finds its tile arrays inside that workspace.  plan() allocates (it is not
part of a captured graph in the reference either, flashomni/attention.py:140-141); run() does not.
"""
import collections
import weakref

import torch

from . import _lib
from .attention import PlannedBatch
from .gemm import _gemm_workspace

_LIB = torch.library.Library("flashomni_kernels", "FRAGMENT")
_MAX_PLANS = 64
_plans = collections.OrderedDict()  # (device index, int workspace address) -> PlannedBatch


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)  # the reference's TORCH_CHECK failures surface as RuntimeError


# ---- attention -------------------------------------------------------------------------------------
def batch_sparseFA_with_kv_plan(float_workspace_buffer, int_workspace_buffer,
                                page_locked_int_workspace_buffer, qo_indptr, kv_indptr, kv_len_arr,
                                total_num_rows, batch_size, num_qo_heads, num_kv_heads, page_size,
                                enable_cuda_graph, head_dim_qk, head_dim_vo):
    """reference: BatchSparseFAWithKVPlan, csrc/batch_sparseFA.cu:39-65.  qo_indptr / kv_indptr are
    host int32 tensors; returns the 15-entry plan vector (CPU int64)."""
    dev = float_workspace_buffer.device
    _check(dev.type == "cuda" and int_workspace_buffer.device == dev,
           "batch_sparseFA_with_kv_plan: the workspaces must live on one GPU")
    _check(qo_indptr.device.type == "cpu" and kv_indptr.device.type == "cpu",
           "batch_sparseFA_with_kv_plan: qo_indptr and kv_indptr are host tensors")
    qo_host = qo_indptr.to(torch.int32).contiguous()
    kv_host = kv_indptr.to(torch.int32).contiguous()
    _check(qo_host.numel() == batch_size + 1 and kv_host.numel() == batch_size + 1,
           "batch_sparseFA_with_kv_plan: indptr arrays must have batch_size + 1 entries")
    _check(head_dim_qk == 128 and head_dim_vo == 128, "only head_dim 128 is supported")
    _check(num_kv_heads > 0 and num_qo_heads % num_kv_heads == 0,
           "num_qo_heads must be a multiple of num_kv_heads")
    plan_info = torch.empty(15, dtype=torch.int64)
    nbytes = lambda t: t.numel() * t.element_size()
    with _lib.device_guard(dev):
        try:
            _lib.check(_lib.lib().fo_prefill_plan(
                _lib.ptr(float_workspace_buffer), nbytes(float_workspace_buffer),
                _lib.ptr(int_workspace_buffer), _lib.ptr(page_locked_int_workspace_buffer),
                nbytes(int_workspace_buffer), _lib.ptr(qo_host), _lib.ptr(kv_host), total_num_rows,
                batch_size, num_qo_heads, num_kv_heads, head_dim_qk, head_dim_vo, page_size,
                int(bool(enable_cuda_graph)), 2, 0, _lib.ptr(plan_info), _lib.current_stream(dev)))
        except RuntimeError as e:  # same wording as csrc/batch_sparseFA.cu:61
            raise RuntimeError("Failed to plan prefill with error: " + str(e)) from None
    key = (dev.index, int_workspace_buffer.data_ptr())
    old = _plans.pop(key, None)
    if old is None:
        # the plan goes when the workspace's memory does: another tensor at the same address later must
        # not find it
        weakref.finalize(int_workspace_buffer.untyped_storage(), _plans.pop, key, None)
    _plans[key] = PlannedBatch(float_workspace_buffer, qo_host, kv_host, qo_host.to(dev), kv_host.to(dev),
                               num_qo_heads, num_kv_heads, 128, 128,
                               worklist=old.worklist if old is not None else None,
                               # grouped-query attention: the reference's symbols, one bit per (tile of
                               # 128 packed rows, kv head) (prefill.cuh:1283-1290)
                               gqa_packed=True)
    _plans[key].plan_vec = plan_info.tolist()
    while len(_plans) > _MAX_PLANS:
        _plans.popitem(last=False)
    return plan_info


def batch_sparseFA_with_ragged_kv_run(float_workspace_buffer, int_workspace_buffer, plan_info_vec, q, k, v,
                                      sparse_info, sparse_kv_info, sparse_info_indptr,
                                      sparse_kv_info_indptr, sparse_block_size_for_q,
                                      sparse_block_size_for_kv, is_full, qo_indptr, kv_indptr, o, maybe_lse,
                                      mask_mode_code, layout, maybe_custom_mask, maybe_mask_indptr,
                                      maybe_alibi_slopes, logits_soft_cap, sm_scale, rope_rcp_scale,
                                      rope_rcp_theta):
    """reference: BatchSparseFAWithRaggedKVRun, csrc/batch_sparseFA.cu:67-201 (argument order as
    flashomni/attention.py:81-138 passes them)."""
    dev = q.device
    pb = _plans.get((dev.index, int_workspace_buffer.data_ptr()))
    _check(pb is not None, "batch_sparseFA_with_ragged_kv_run: no plan was made with this int workspace "
                           "(call batch_sparseFA_with_kv_plan first)")
    # (the vector is what the caller got from that plan call: a workspace planned again since, by
    # another owner, holds another batch's tables)
    _check(list(plan_info_vec.tolist() if torch.is_tensor(plan_info_vec) else plan_info_vec) == pb.plan_vec,
           "batch_sparseFA_with_ragged_kv_run: plan_info_vec is not the plan last made with this int "
           "workspace")
    _check(q.dim() == 3 and q.size(1) == pb.num_qo_heads,
           "batch_sparseFA_with_ragged_kv_run: q does not have the planned number of heads")
    _check(mask_mode_code == 0 and maybe_custom_mask is None and maybe_mask_indptr is None,
           "only the non-causal mask mode is built (as in the reference's shipped kernels)")
    _check(maybe_alibi_slopes is None, "ALiBi is not built (as in the reference's shipped kernels)")
    _check(0.0 <= logits_soft_cap < float("inf"), "logits_soft_cap must be a finite value >= 0")
    _check(sparse_block_size_for_q == 128 and sparse_block_size_for_kv == 128,
           "only 128 x 128 sparse blocks are supported")
    _check(layout in (0, 1), "layout must be 0 (NHD) or 1 (HND)")
    _check(q.dtype in (torch.bfloat16, torch.float16) and k.dtype == q.dtype and v.dtype == q.dtype
           and o.dtype == q.dtype, "q, k, v and o must share one 16-bit float dtype")
    _check(o.shape == q.shape and o.device == dev, "o must have q's shape and device")
    for name, t in (("qo_indptr", qo_indptr), ("kv_indptr", kv_indptr)):
        _check(t.device == dev and t.dtype == torch.int32 and t.is_contiguous()
               and t.numel() == pb.batch_size + 1,
               "%s must be the planned batch's int32 indptr on the GPU" % name)
    if maybe_lse is not None:
        _check(maybe_lse.shape == (q.size(0), q.size(1)) and maybe_lse.dtype == torch.float32
               and maybe_lse.device == dev, "lse must be float32 [nnz_q, num_qo_heads] on q's device")
    if pb.float_ws.data_ptr() != float_workspace_buffer.data_ptr() or \
            pb.float_ws.numel() != float_workspace_buffer.numel():
        pb.float_ws = float_workspace_buffer
        pb.split_ok = pb._split_ws_ok()
    pb.qo_indptr, pb.kv_indptr = qo_indptr, kv_indptr
    try:
        pb.decode(sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr, is_full)
        pb.launch(q, k, v, o, maybe_lse, "NHD" if layout == 0 else "HND", sm_scale,
                  logits_soft_cap=logits_soft_cap)
    except ValueError as e:
        raise RuntimeError(str(e)) from None


# ---- GEMMs -----------------------------------------------------------------------------------------
def _gemm_shapes(x, w, y, name):
    _check(x.dim() == 3 and w.dim() == 2 and y.dim() == 3, name + ": x [B,M,K], w [N,K], y [B,M,N]")
    _check(x.size(0) == y.size(0), "Batch sizes must match")          # csrc/gemm.cu:32
    _check(x.size(1) == y.size(1), "Token sizes must match")          # :33
    _check(x.size(2) == w.size(1) and w.size(0) == y.size(2), "Result tensor has incorrect shape")  # :34-35
    _check(x.is_cuda and w.device == x.device and y.device == x.device, name + ": tensors must share one GPU")
    _check(x.dtype in (torch.bfloat16, torch.float16) and w.dtype == x.dtype,
           name + ": x and w must both be bfloat16 or float16")
    _check(x.is_contiguous() and w.is_contiguous() and y.is_contiguous(), name + ": tensors must be contiguous")


def _symbol_args(info, indptr, dev, name, batch):
    if info is None:
        return None, None
    _check(indptr is not None, name + ": sparse_info needs sparse_info_indptr")
    _check(info.device == dev and indptr.device == dev, name + ": symbols must be on x's device")
    if info.dtype != torch.uint8 or not info.is_contiguous():
        info = info.to(torch.uint8).contiguous()
    if indptr.dtype != torch.int32 or not indptr.is_contiguous():
        indptr = indptr.to(torch.int32).contiguous()
    _check(indptr.numel() == batch + 1, name + ": sparse_info_indptr must have batch + 1 entries")
    return info, indptr


def flashomni_gemm(x, w, y, bias, sparse_q_size, num_qo_heads, sparse_info, sparse_info_indptr,
                   num_text_tokens, is_full):
    """reference: FLASHOMNIGEMM, csrc/gemm.cu:24-59 (M may have a tail here)."""
    _gemm_shapes(x, w, y, "flashomni_gemm")
    _check(y.dtype == x.dtype, "flashomni_gemm: y must have x's dtype")
    B, M, K = x.shape
    N = w.size(0)
    _check(num_qo_heads > 0 and N % num_qo_heads == 0, "flashomni_gemm: N must be a multiple of num_qo_heads")
    if bias is not None:
        _check(bias.dtype == x.dtype and bias.numel() == N and bias.device == x.device,
               "flashomni_gemm: bias must be [N] with x's dtype on x's device")
        bias = bias.contiguous()
    info, indptr = (None, None) if is_full else _symbol_args(sparse_info, sparse_info_indptr, x.device,
                                                             "flashomni_gemm", B)
    _check(is_full or info is not None, "flashomni_gemm: sparse_info is required unless is_full")
    if info is not None and M > 0:
        need = (((num_text_tokens + M - 1) // sparse_q_size + 1) * num_qo_heads + 7) // 8
        _check(info.numel() >= need, "flashomni_gemm: sparse_info is shorter than the bits the tiles read")
    L = _lib.lib()
    ws_bytes = L.fo_gemm_workspace_bytes(B, M, N)
    stream = _lib.current_stream(x.device)
    ws = _gemm_workspace(x.device, stream, ws_bytes)
    with _lib.device_guard(x.device):
        _lib.check(L.fo_gemm_q(_lib.ptr(x), _lib.ptr(w), _lib.ptr(bias), _lib.ptr(y), _lib.dtype_code(x.dtype),
                               B, M, N, K, sparse_q_size, num_qo_heads, _lib.ptr(info), _lib.ptr(indptr),
                               num_text_tokens, int(bool(is_full)), _lib.ptr(ws), ws_bytes, stream))


def flashomni_gemm_reduction(x, w, y, bias, sparse_q_size, num_qo_heads, sparse_info, sparse_info_indptr,
                             num_text_tokens, is_for_cached):
    """reference: FLASHOMNIGEMMReduction, csrc/gemm_reduction.cu:24-57.  bias is the vector [N] when
    is_for_cached, else the cached partial [B,M,N] (gemm_reduction.cuh:77-95)."""
    _gemm_shapes(x, w, y, "flashomni_gemm_reduction")
    _check(y.dtype in (x.dtype, torch.float32), "flashomni_gemm_reduction: y must have x's dtype or float32")
    B, M, K = x.shape
    N = w.size(0)
    _check(num_qo_heads > 0, "flashomni_gemm_reduction: num_qo_heads > 0 is required")
    kind, bias_code = _lib.FO_BIAS_NONE, _lib.dtype_code(x.dtype)
    if bias is not None:
        _check(bias.device == x.device, "flashomni_gemm_reduction: bias must be on x's device")
        if is_for_cached:
            _check(bias.numel() == N and bias.dtype == x.dtype,
                   "flashomni_gemm_reduction: with is_for_cached bias must be [N] with x's dtype")
            kind = _lib.FO_BIAS_VECTOR
        else:
            _check(bias.numel() == B * M * N and bias.dtype in (x.dtype, torch.float32),
                   "flashomni_gemm_reduction: without is_for_cached bias must be the cached [B, M, N] partial")
            kind, bias_code = _lib.FO_BIAS_MATRIX, _lib.dtype_code(bias.dtype)
        bias = bias.contiguous()
    info, indptr = _symbol_args(sparse_info, sparse_info_indptr, x.device, "flashomni_gemm_reduction", B)
    _check(info is not None, "flashomni_gemm_reduction: sparse_info is required")
    if M > 0:
        need = (((num_text_tokens + M - 1) // sparse_q_size + 1) * num_qo_heads + 7) // 8
        _check(info.numel() >= need, "flashomni_gemm_reduction: sparse_info is shorter than the bits the tiles read")
    stream = _lib.current_stream(x.device)
    ws = _gemm_workspace(x.device, stream, 256)  # work-item cursors of a long launch
    with _lib.device_guard(x.device):
        _lib.check(_lib.lib().fo_gemm_o(
            _lib.ptr(x), _lib.ptr(w), _lib.ptr(bias), _lib.ptr(y), _lib.dtype_code(x.dtype), kind, bias_code,
            _lib.dtype_code(y.dtype), B, M, N, K, sparse_q_size, num_qo_heads, _lib.ptr(info),
            _lib.ptr(indptr), num_text_tokens, int(bool(is_for_cached)), _lib.ptr(ws), 256, stream))


# ---- bit packing -----------------------------------------------------------------------------------
def _bitorder(bitorder):
    _check(bitorder in ("big", "little"), "bitorder must be 'big' or 'little'")  # csrc/quantization.cu:25
    return 0 if bitorder == "big" else 1


def _bool_bytes(x):
    _check(x.is_cuda and x.is_contiguous(), "x must be a contiguous GPU tensor")  # CHECK_INPUT, :23
    if x.dtype == torch.bool:
        return x.view(torch.uint8)
    return x.to(torch.bool).view(torch.uint8)


def packbits(x, bitorder, y):
    """reference: packbits, csrc/quantization.cu:22-36."""
    code = _bitorder(bitorder)
    xb = _bool_bytes(x)
    _check(y.dtype == torch.uint8 and y.device == x.device and y.is_contiguous()
           and y.numel() >= (xb.numel() + 7) // 8, "y must be uint8 with (numel(x) + 7) // 8 bytes on x's device")
    with _lib.device_guard(x.device):
        _lib.check(_lib.lib().fo_packbits(_lib.ptr(xb), xb.numel(), code, _lib.ptr(y),
                                          _lib.current_stream(x.device)))


def segment_packbits(x, input_indptr, output_indptr, bitorder, y):
    """reference: segment_packbits, csrc/quantization.cu:38-57."""
    code = _bitorder(bitorder)
    xb = _bool_bytes(x)
    for t in (input_indptr, output_indptr):
        _check(t.device == x.device and t.is_contiguous() and t.dtype == torch.int32,
               "indptr arrays must be contiguous int32 tensors on x's device")
    _check(output_indptr.numel() == input_indptr.numel() and input_indptr.numel() >= 1,
           "input_indptr and output_indptr must have batch_size + 1 entries")
    _check(y.dtype == torch.uint8 and y.device == x.device and y.is_contiguous(), "y must be uint8 on x's device")
    with _lib.device_guard(x.device):
        _lib.check(_lib.lib().fo_segment_packbits(_lib.ptr(xb), _lib.ptr(input_indptr), _lib.ptr(output_indptr),
                                                  input_indptr.numel() - 1, code, _lib.ptr(y),
                                                  _lib.current_stream(x.device)))


_SCHEMAS = (
    ("batch_sparseFA_with_kv_plan",
     "(Tensor float_workspace_buffer, Tensor int_workspace_buffer, Tensor page_locked_int_workspace_buffer, "
     "Tensor qo_indptr, Tensor kv_indptr, Tensor kv_len_arr, int total_num_rows, int batch_size, "
     "int num_qo_heads, int num_kv_heads, int page_size, bool enable_cuda_graph, int head_dim_qk, "
     "int head_dim_vo) -> Tensor", batch_sparseFA_with_kv_plan),
    ("batch_sparseFA_with_ragged_kv_run",
     "(Tensor(a!) float_workspace_buffer, Tensor(b!) int_workspace_buffer, Tensor plan_info_vec, Tensor q, "
     "Tensor k, Tensor v, Tensor? sparse_info, Tensor? sparse_kv_info, Tensor? sparse_info_indptr, "
     "Tensor? sparse_kv_info_indptr, int sparse_block_size_for_q, int sparse_block_size_for_kv, bool is_full, "
     "Tensor qo_indptr, Tensor kv_indptr, Tensor(c!) o, Tensor(d!)? maybe_lse, int mask_mode_code, int layout, "
     "Tensor? maybe_custom_mask, Tensor? maybe_mask_indptr, Tensor? maybe_alibi_slopes, float logits_soft_cap, "
     "float sm_scale, float rope_rcp_scale, float rope_rcp_theta) -> ()", batch_sparseFA_with_ragged_kv_run),
    ("flashomni_gemm",
     "(Tensor x_ptr, Tensor w_ptr, Tensor(a!) y_ptr, Tensor? bias, int sparse_q_size, int num_qo_heads, "
     "Tensor? sparse_info, Tensor? sparse_info_indptr, int num_text_tokens, bool is_full) -> ()", flashomni_gemm),
    ("flashomni_gemm_reduction",
     "(Tensor x_ptr, Tensor w_ptr, Tensor(a!) y_ptr, Tensor? bias, int sparse_q_size, int num_qo_heads, "
     "Tensor sparse_info, Tensor sparse_info_indptr, int num_text_tokens, bool is_for_cached) -> ()",
     flashomni_gemm_reduction),
    ("packbits", "(Tensor x, str bitorder, Tensor(a!) y) -> ()", packbits),
    ("segment_packbits",
     "(Tensor x, Tensor input_indptr, Tensor output_indptr, str bitorder, Tensor(a!) y) -> ()", segment_packbits),
)
OP_NAMES = tuple(name for name, _, _ in _SCHEMAS)

for _name, _schema, _fn in _SCHEMAS:
    _LIB.define(_name + _schema)
    _LIB.impl(_name, _fn, "CompositeExplicitAutograd")
