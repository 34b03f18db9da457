"""``BatchFlashOmniFAWithRaggedKVWrapper``: ragged block-sparse FlashAttention prefill.

The public surface (constructor, ``plan``, ``run``, ``run_return_lse``, the deprecated
``forward*`` aliases, defaults and error types) is that of the reference
(flashomni/attention.py:194-869).  Behind it:

* ``plan()`` runs the host planner (fo_prefill_plan) into the wrapper's integer workspace, builds
  the q-block table and sizes the work-list buffers;
* ``run()`` first decodes the bit-packed symbols into a compacted work list on the GPU
  (fo_decode_sparse, every call: the symbol buffers may have been rewritten in place by writers
  torch does not see; ``reuse_decoded=True`` skips it on the caller's word) and then launches the
  sparse FlashAttention kernel over that list (fo_sparse_fa_run).

Of the options the reference's shipped build supports (setup.py:30-38, :98-111) head_dim 128 and the
logits soft cap are implemented: no causal / custom mask, no positional encoding, fp32 logits.
"""
import functools
import math
from typing import Optional, Tuple, Union

import torch

from . import _lib
from .utils import (MaskMode, PosEncodingMode, TensorLayout, _check_cached_qkv_data_type,  # noqa: F401
                    _check_kv_layout, _check_pos_encoding_mode, _check_shape_dtype_device,
                    canonicalize_torch_dtype, is_float8)


def _compute_sparse_info_indptr(qo_indptr: torch.Tensor, num_qo_heads, sparse_block_size_for_q: int,
                                device: torch.device = "cuda") -> torch.Tensor:
    """Bit-count indptr of ``sparse_info`` (reference: flashomni/attention.py:165-176)."""
    sparse_info_indptr = torch.empty_like(qo_indptr, device=device)
    sparse_info_indptr[0] = 0
    sparse_info_indptr[1:] = torch.cumsum(
        torch.ceil((qo_indptr[1:] - qo_indptr[:-1]) / sparse_block_size_for_q) * num_qo_heads, 0)
    return sparse_info_indptr


def _compute_sparse_kv_info_indptr(qo_indptr: torch.Tensor, kv_indptr: torch.Tensor, num_qo_heads,
                                   sparse_block_size_for_q: int, sparse_block_size_for_kv: int,
                                   device: torch.device = "cuda") -> torch.Tensor:
    """Bit-count indptr of ``sparse_kv_info`` (reference: flashomni/attention.py:178-191)."""
    sparse_kv_info_indptr = torch.empty_like(qo_indptr, device=device)
    sparse_kv_info_indptr[0] = 0
    sparse_kv_info_indptr[1:] = torch.cumsum(
        torch.ceil((qo_indptr[1:] - qo_indptr[:-1]) / sparse_block_size_for_q)
        * torch.ceil((kv_indptr[1:] - kv_indptr[:-1]) / sparse_block_size_for_kv)
        * num_qo_heads, 0)
    return sparse_kv_info_indptr


class DecodedWorkList:
    """Device buffers holding one decoded work list (canonical order).

    ``row_req/row_qb/row_head[n_rows]``, ``kv_row_ptr[n_rows+1]``, ``kv_idx[nnz]``, all int32;
    ``counts = [n_rows, nnz, 0, 0]``; ``order[n_rows]`` / ``sched[1024]`` are the execution order
    and queue words the attention kernel schedules from; ``shares`` holds one record per queue
    entry or, when there are only a few rows per CU, the table of even shares used instead.  The sizes live on the device;
    ``sizes()`` copies them back (one synchronisation) for tests and reports."""

    def __init__(self, max_rows: int, max_nnz: int, num_heads: int, device):
        self.max_rows, self.max_nnz = max_rows, max_nnz
        n = max(max_rows, 1)
        self.row_req = torch.empty(n, dtype=torch.int32, device=device)
        self.row_qb = torch.empty(n, dtype=torch.int32, device=device)
        self.row_head = torch.empty(n, dtype=torch.int32, device=device)
        self.kv_row_ptr = torch.empty(n + 1, dtype=torch.int32, device=device)
        self.kv_idx = torch.empty(max(max_nnz, 1), dtype=torch.int32, device=device)
        self.counts = torch.zeros(4, dtype=torch.int32, device=device)
        self.order = torch.empty(n, dtype=torch.int32, device=device)
        self.sched = torch.zeros(1024, dtype=torch.int32, device=device)
        self.shares = torch.zeros(512 + 8 * (n + 1), dtype=torch.int32, device=device)
        self.scratch = torch.empty(2 * n + 8192, dtype=torch.int32, device=device)

    def sizes(self) -> Tuple[int, int]:
        c = self.counts.cpu()
        return int(c[0]), int(c[1])

    def to_host(self):
        n_rows, nnz = self.sizes()
        return (self.row_req[:n_rows].cpu(), self.row_qb[:n_rows].cpu(), self.row_head[:n_rows].cpu(),
                self.kv_row_ptr[:n_rows + 1].cpu(), self.kv_idx[:nnz].cpu())


class PlannedBatch:
    """Everything ``plan`` derives from a ragged batch beyond the reference planner's arrays: the
    decoder's q-block table, the block numbering of the fp8 scales, the sizes ``run`` checks its
    tensors against and the work-list buffers (sized for the all-ones worst case).  Shared by the
    wrapper and by the ``torch.ops.flashomni_kernels`` operators, which have no slot for these
    buffers in the reference's signatures and look the object up by their integer workspace."""

    def __init__(self, float_workspace_buffer, qo_indptr_host, kv_indptr_host, qo_indptr_dev,
                 kv_indptr_dev, num_qo_heads, num_kv_heads, block_q, block_kv, share_rows=True,
                 worklist=None, gqa_packed=False):
        L = _lib.lib()
        self.device = float_workspace_buffer.device
        self.float_ws = float_workspace_buffer
        self.qo_indptr, self.kv_indptr = qo_indptr_dev, kv_indptr_dev
        self.num_qo_heads, self.num_kv_heads = num_qo_heads, num_kv_heads
        self.block_q, self.block_kv = block_q, block_kv
        batch_size = qo_indptr_host.numel() - 1
        self.batch_size = batch_size
        # What a work-list row is.  Packed (the reference's layout for grouped-query attention,
        # include/flashomni/attention/prefill.cuh:410-413, 1283-1290): a request's q rows are its
        # (token, q head of the group) pairs, token-major; a row is (request, tile of 128 pairs, kv
        # head) and the symbols hold one bit per (tile, kv head).  For the decoder that is a batch
        # whose requests are `group` times as long, with num_kv_heads heads.
        self.gqa_packed = bool(gqa_packed) and num_kv_heads != num_qo_heads
        self.symbol_heads = num_kv_heads if self.gqa_packed else num_qo_heads
        qo_rows_host = qo_indptr_host
        if self.gqa_packed:
            rows = qo_indptr_host.to(torch.int64) * (num_qo_heads // num_kv_heads)
            if int(rows[-1]) >= 2 ** 31:
                raise RuntimeError("Failed to plan prefill with error: too many packed q rows")
            qo_rows_host = rows.to(torch.int32).contiguous()
        n_blk = torch.zeros(3, dtype=torch.int64)
        _lib.check(L.fo_decode_sizes(_lib.ptr(qo_rows_host), _lib.ptr(kv_indptr_host), batch_size,
                                     self.symbol_heads, block_q, block_kv,
                                     n_blk[0:].data_ptr(), n_blk[1:].data_ptr(), n_blk[2:].data_ptr()))
        n_q_blk, max_rows, max_nnz = (int(v) for v in n_blk)
        if max_nnz >= 2 ** 31:
            raise RuntimeError("Failed to plan prefill with error: work list too large")
        table = torch.empty((2, max(n_q_blk, 1)), dtype=torch.int32)
        _lib.check(L.fo_sparse_block_table(_lib.ptr(qo_rows_host), batch_size, block_q,
                                           table[0].data_ptr(), table[1].data_ptr(), n_q_blk,
                                           n_blk[0:].data_ptr()))
        self.blk_table = table.to(self.device)
        self.n_q_blk = n_q_blk
        qlen = (qo_indptr_host[1:] - qo_indptr_host[:-1]).to(torch.int64)
        klen = (kv_indptr_host[1:] - kv_indptr_host[:-1]).to(torch.int64)
        q_base = torch.zeros(batch_size + 1, dtype=torch.int64)
        kv_base = torch.zeros(batch_size + 1, dtype=torch.int64)
        q_base[1:] = torch.cumsum((qlen + block_q - 1) // block_q, 0)
        kv_base[1:] = torch.cumsum((klen + block_kv - 1) // block_kv, 0)
        self.q_blk_base = q_base.to(torch.int32).to(self.device)
        self.kv_blk_base = kv_base.to(torch.int32).to(self.device)
        self.n_kv_blk = int(kv_base[-1])
        self.max_kv_len = int(klen.max()) if klen.numel() else 0
        # sizes the tensors given to run() must have (checked there without reading the device):
        # token counts, and the packed bytes of the byte-aligned per-request segments
        self.total_q_rows = int(qo_indptr_host[-1]) if qo_indptr_host.numel() else 0
        self.total_kv_rows = int(kv_indptr_host[-1]) if kv_indptr_host.numel() else 0
        qrows = (qo_rows_host[1:] - qo_rows_host[:-1]).to(torch.int64)
        nqb = (qrows + block_q - 1) // block_q   # symbol rows (q blocks or packed tiles) per request
        nkb = kv_base[1:] - kv_base[:-1]
        self.min_info_bytes = int(((nqb * self.symbol_heads + 7) // 8).sum())
        self.min_kv_info_bytes = int(((nqb * nkb * self.symbol_heads + 7) // 8).sum())
        if worklist is None or worklist.max_rows < max_rows or worklist.max_nnz < max_nnz:
            worklist = DecodedWorkList(max_rows, max_nnz, self.symbol_heads, self.device)
        self.worklist = worklist
        self.max_rows = max_rows
        self.share_rows = share_rows
        self.split_ok = self._split_ws_ok()
        # [is_full, stream, streams already ordered after it] of the list the work-list buffers hold
        self.decoded = None

    def float_ws_bytes(self) -> int:
        return self.float_ws.numel() * self.float_ws.element_size()

    def _split_ws_ok(self) -> bool:
        """Whether the float workspace can hold the partial results of rows whose kv list is shared
        between workgroups (the reference uses it for its split-kv partials, scheduler.cuh:322-328)."""
        return (self.share_rows and self.float_ws.data_ptr() % 16 == 0
                and self.float_ws_bytes() >= _lib.lib().fo_sparse_fa_split_workspace_bytes())

    def decode(self, sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr,
               is_full: bool = False) -> DecodedWorkList:
        """fo_decode_sparse on the current stream into the work-list buffers."""
        wl = self.worklist
        if not is_full:
            if sparse_info is None or sparse_kv_info is None or sparse_info_indptr is None \
                    or sparse_kv_info_indptr is None:
                raise ValueError("sparse_info, sparse_kv_info and their indptrs are required unless "
                                 "is_full=True")
            tensors = []
            for name, t, dt in (("sparse_info", sparse_info, torch.uint8),
                                ("sparse_kv_info", sparse_kv_info, torch.uint8),
                                ("sparse_info_indptr", sparse_info_indptr, torch.int32),
                                ("sparse_kv_info_indptr", sparse_kv_info_indptr, torch.int32)):
                if t.device != self.device:
                    raise ValueError(f"Invalid device of {name}: expected {self.device}, got {t.device}")
                if t.dtype != dt or not t.is_contiguous():
                    t = t.to(dt).contiguous()
                tensors.append(t)
            for name, t, need in (("sparse_info", tensors[0], self.min_info_bytes),
                                  ("sparse_kv_info", tensors[1], self.min_kv_info_bytes)):
                if t.numel() < need:
                    raise ValueError(f"{name} holds {t.numel()} bytes; the planned batch needs {need}")
            for name, t in (("sparse_info_indptr", tensors[2]), ("sparse_kv_info_indptr", tensors[3])):
                if t.numel() != self.batch_size + 1:
                    raise ValueError(f"{name} must have {self.batch_size + 1} entries, got {t.numel()}")
        else:
            tensors = [None] * 4
        stream = torch.cuda.current_stream(self.device)
        with _lib.device_guard(self.device):
            _lib.check(_lib.lib().fo_decode_sparse(
                _lib.ptr(tensors[0]), _lib.ptr(tensors[1]), _lib.ptr(tensors[2]), _lib.ptr(tensors[3]),
                _lib.ptr(self.blk_table[0]), _lib.ptr(self.blk_table[1]), _lib.ptr(self.kv_indptr),
                self.n_q_blk, self.symbol_heads, self.block_kv, int(bool(is_full)),
                _lib.ptr(wl.row_req), _lib.ptr(wl.row_qb), _lib.ptr(wl.row_head), _lib.ptr(wl.kv_row_ptr),
                _lib.ptr(wl.kv_idx), _lib.ptr(wl.counts), _lib.ptr(wl.order), _lib.ptr(wl.sched),
                _lib.ptr(wl.scratch), _lib.ptr(wl.shares if self.split_ok else None),
                stream.cuda_stream))
        # remembered for reuse_decoded: which stream the list was decoded on (a run on another
        # stream must be ordered after it)
        self.decoded = (bool(is_full), stream, [])
        return wl

    def reuse_decoded(self, is_full: bool) -> DecodedWorkList:
        """The work list of the last decode, ordered before the current stream's work."""
        if self.decoded is None:
            raise RuntimeError("reuse_decoded=True needs an earlier decode() or run() after plan()")
        was_full, stream, ordered = self.decoded
        if was_full != bool(is_full):
            raise RuntimeError("reuse_decoded=True: the last decode was made with is_full=%s" % was_full)
        cur = torch.cuda.current_stream(self.device)
        # one wait per (decode, stream): later work on a stream that has waited is behind the decode
        # already, and a wait in front of every launch costs each one 2-3 us
        if cur != stream and cur not in ordered and not torch.cuda.is_current_stream_capturing():
            ev = torch.cuda.Event()
            ev.record(stream)
            cur.wait_event(ev)
            ordered.append(cur)
        return self.worklist

    def launch(self, q, k, v, out, lse, kv_layout, sm_scale, q_scale=None, k_scale=None, q_lo=None,
               k_lo=None, logits_soft_cap=0.0) -> None:
        """Shape checks against the planned batch, then fo_sparse_fa_run over the decoded list."""
        if logits_soft_cap and logits_soft_cap > 0 and is_float8(q):
            raise NotImplementedError("the logits soft cap takes 16-bit q and k")
        if q.dim() != 3 or k.dim() != 3 or v.dim() != 3 or k.size(2) != 128 or v.size(2) != 128:
            raise ValueError("q, k and v must be 3-dimensional with head_dim 128")
        fp8 = is_float8(q)
        if fp8 and self.gqa_packed:
            raise NotImplementedError(
                "fp8 q has one scale per (q head, 128-token block); packed tiles of several q heads "
                "(grouped-query attention in the reference's symbol layout) take 16-bit q and k")
        if fp8:
            if q.dtype != torch.float8_e4m3fn or k.dtype != torch.float8_e4m3fn \
                    or q_scale is None or k_scale is None:
                raise ValueError("fp8 attention needs float8_e4m3fn q and k with q_scale and k_scale")
            if v.dtype != torch.bfloat16:
                raise ValueError("fp8 attention keeps v (and the output) in bfloat16")
            if q_lo is not None and (q_lo.dtype != q.dtype or q_lo.shape != q.shape
                                     or q_lo.stride() != q.stride() or q_lo.device != q.device):
                raise ValueError("q_lo must be a float8_e4m3fn tensor laid out like q")
            if k_lo is not None and (k_lo.dtype != k.dtype or k_lo.shape != k.shape
                                     or k_lo.stride() != k.stride() or k_lo.device != k.device):
                raise ValueError("k_lo must be a float8_e4m3fn tensor laid out like k")
            if k_lo is not None and q_lo is None:
                raise ValueError("k_lo (the second term of an fp8 k) needs q_lo as well")
            if k_lo is not None and self.max_kv_len > 2048 * 128:
                raise NotImplementedError("with k_lo a request may hold at most 262144 kv tokens")
        elif q_lo is not None or k_lo is not None:
            raise ValueError("q_lo / k_lo are the second terms of an fp8 q / k")
        if q.device != self.device:
            raise ValueError(f"Invalid device of q: expected {self.device}, got {q.device}")
        if q.size(1) != self.num_qo_heads or q.size(2) != 128:
            raise ValueError("q does not match the head count / head_dim given to plan()")
        kv_head_dim = 1 if kv_layout == "NHD" else 0
        if k.size(kv_head_dim) != self.num_kv_heads or v.size(kv_head_dim) != self.num_kv_heads:
            raise ValueError("k / v do not match the kv head count given to plan()")
        n_kv = min(k.size(1 - kv_head_dim), v.size(1 - kv_head_dim))
        if q.size(0) < self.total_q_rows or n_kv < self.total_kv_rows:
            raise ValueError(f"q / k, v hold {q.size(0)} / {n_kv} tokens; the planned "
                             f"batch has {self.total_q_rows} / {self.total_kv_rows}")
        if lse is not None and not lse.is_contiguous():
            raise ValueError("lse must be contiguous")
        for name, t in (("q", q), ("k", k), ("v", v), ("out", out)):
            if t.stride(-1) != 1:
                raise ValueError(f"{name} must have a contiguous last dimension")
        if kv_layout == "NHD":
            k_sn, k_sh, v_sn, v_sh = k.stride(0), k.stride(1), v.stride(0), v.stride(1)
        else:
            k_sh, k_sn, v_sh, v_sn = k.stride(0), k.stride(1), v.stride(0), v.stride(1)
        if fp8:
            q_scale = q_scale.to(torch.float32).contiguous()
            k_scale = k_scale.to(torch.float32).contiguous()
            if q_scale.shape != (q.size(1), self.n_q_blk) or \
                    k_scale.shape != (self.num_kv_heads, self.n_kv_blk):
                raise ValueError("q_scale / k_scale must be [H, number of 128-token blocks] "
                                 "(k_scale: one row per kv head)")
        wl = self.worklist
        with _lib.device_guard(self.device):
            _lib.check(_lib.lib().fo_sparse_fa_run(
                _lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(out), _lib.ptr(lse),
                _lib.dtype_code(q.dtype), _lib.ptr(q_lo), _lib.ptr(k_lo), _lib.ptr(q_scale if fp8 else None),
                _lib.ptr(k_scale if fp8 else None),
                q.stride(0), q.stride(1), k_sn, k_sh, v_sn, v_sh, out.stride(0), out.stride(1),
                _lib.ptr(self.qo_indptr), _lib.ptr(self.kv_indptr), _lib.ptr(self.q_blk_base),
                _lib.ptr(self.kv_blk_base), self.n_q_blk, self.n_kv_blk, _lib.ptr(wl.row_req),
                _lib.ptr(wl.row_qb), _lib.ptr(wl.row_head), _lib.ptr(wl.kv_row_ptr), _lib.ptr(wl.kv_idx),
                _lib.ptr(wl.order), _lib.ptr(wl.sched), self.max_rows, q.size(1), self.num_kv_heads,
                int(self.gqa_packed), q.size(2), self.block_q, self.block_kv, float(sm_scale),
                float(logits_soft_cap or 0.0),
                _lib.ptr(wl.shares if self.split_ok else None),
                _lib.ptr(self.float_ws) if self.split_ok else None,
                self.float_ws_bytes(), _lib.current_stream(self.device)))


class BatchFlashOmniFAWithRaggedKVWrapper:
    r"""Wrapper class for block-sparse prefill attention over ragged q/k/v tensors.

    >>> workspace = torch.empty(128 * 1024 * 1024, dtype=torch.uint8, device="cuda:0")
    >>> wrapper = BatchFlashOmniFAWithRaggedKVWrapper(workspace, "NHD")
    >>> wrapper.plan(qo_indptr, kv_indptr, num_qo_heads, num_kv_heads, head_dim,
    ...              sparse_block_size_for_q=128, sparse_block_size_for_kv=128,
    ...              q_data_type=torch.bfloat16)
    >>> o = wrapper.run(q, k, v, sparse_info, sparse_kv_info, sparse_info_indptr,
    ...                 sparse_kv_info_indptr)

    ``sparse_info`` holds one bit per (q-block, head) (1 = compute, 0 = cached: the rows of ``out``
    are left untouched), ``sparse_kv_info`` one bit per (q-block, head, kv-block) (1 = keep), both
    packed little-endian per request; the two indptr tensors are the byte offsets returned by
    ``segment_packbits``.
    """

    def __init__(
        self,
        float_workspace_buffer: torch.Tensor,
        kv_layout: str = "NHD",
        use_cuda_graph: bool = False,
        qo_indptr_buf: Optional[torch.Tensor] = None,
        kv_indptr_buf: Optional[torch.Tensor] = None,
        custom_mask_buf: Optional[torch.Tensor] = None,
        mask_indptr_buf: Optional[torch.Tensor] = None,
        backend: str = "auto",
    ) -> None:
        _check_kv_layout(kv_layout)
        self._kv_layout = kv_layout
        self._float_workspace_buffer = float_workspace_buffer
        # give the decoder a share table (queue-entry records; even shares for short lists); needs a
        # float workspace of fo_sparse_fa_split_workspace_bytes().  Read at plan() time.
        self._share_rows = True
        self.device = float_workspace_buffer.device
        if self.device.type != "cuda":
            raise ValueError("float_workspace_buffer must live on the GPU; there is no CPU path")
        self._int_workspace_buffer = torch.empty((8 * 1024 * 1024,), dtype=torch.uint8,
                                                 device=self.device)
        self._pin_memory_int_workspace_buffer = torch.empty(
            self._int_workspace_buffer.shape, dtype=torch.uint8, pin_memory=True, device="cpu")
        self._use_cuda_graph = use_cuda_graph
        if use_cuda_graph:
            if not torch.is_tensor(qo_indptr_buf):
                raise ValueError("qo_indptr_buf should be a torch.Tensor in cuda graph mode")
            if not torch.is_tensor(kv_indptr_buf):
                raise ValueError("kv_indptr_buf should be a torch.Tensor in cuda graph mode")
            self._fixed_batch_size = len(qo_indptr_buf) - 1
            if len(kv_indptr_buf) != self._fixed_batch_size + 1:
                raise ValueError(
                    "The length of kv_indptr_buf ({}) should be the same as qo_indptr_buf ({}).".format(
                        len(kv_indptr_buf), self._fixed_batch_size))
        self._qo_indptr_buf = qo_indptr_buf
        self._kv_indptr_buf = kv_indptr_buf
        self._custom_mask_buf = custom_mask_buf
        self._mask_indptr_buf = mask_indptr_buf
        self._max_total_num_rows = None
        self._backend = backend  # accepted for compatibility; there is one HIP code path
        self._plan_info = None
        self._planned = None  # PlannedBatch of the last plan()

    @property
    def is_cuda_graph_enabled(self) -> bool:
        return self._use_cuda_graph

    def reset_workspace_buffer(self, float_workspace_buffer: torch.Tensor,
                               int_workspace_buffer) -> None:
        self._float_workspace_buffer = float_workspace_buffer
        self._int_workspace_buffer = int_workspace_buffer
        self._pin_memory_int_workspace_buffer = torch.empty(
            self._int_workspace_buffer.shape, dtype=self._int_workspace_buffer.dtype, device="cpu",
            pin_memory=True)
        # whether rows may be shared between workgroups depends on the float workspace, and a list
        # decoded for the old buffers' share table must not be reused
        if self._planned is not None:
            self._planned.float_ws = float_workspace_buffer
            self._planned.split_ok = self._planned._split_ws_ok()
            self._planned.decoded = None

    # ------------------------------------------------------------------------------------------
    def plan(
        self,
        qo_indptr: torch.Tensor,
        kv_indptr: torch.Tensor,
        num_qo_heads: int,
        num_kv_heads: int,
        head_dim_qk: int,
        sparse_block_size_for_q: int = 128,
        sparse_block_size_for_kv: int = 128,
        head_dim_vo: Optional[int] = None,
        custom_mask: Optional[torch.Tensor] = None,
        packed_custom_mask: Optional[torch.Tensor] = None,
        causal: bool = False,
        pos_encoding_mode: str = "NONE",
        use_fp16_qk_reduction: bool = False,
        logits_soft_cap: Optional[float] = None,
        sm_scale: Optional[float] = None,
        rope_scale: Optional[float] = None,
        rope_theta: Optional[float] = None,
        q_data_type: Union[str, torch.dtype] = "float16",
        kv_data_type: Optional[Union[str, torch.dtype]] = None,
        *,
        gqa_symbols: Optional[str] = None,
    ) -> None:
        r"""Plan sparse prefill attention for the given ragged batch.

        Same parameters as the reference ``plan``, plus ``gqa_symbols`` (keyword-only).  With
        ``num_kv_heads < num_qo_heads`` the reference packs the q heads of a kv head into the row
        dimension (row r of a request = token r // group, q head kv_head * group + r % group,
        include/flashomni/attention/prefill.cuh:410-413) and reads one symbol per (tile of 128
        packed rows, kv head): ``bit = tile * num_kv_heads + kv_head``, followed in
        ``sparse_kv_info`` by one bit per kv block (prefill.cuh:1283-1290).  That is the layout
        read by default (``gqa_symbols=None`` or ``"packed_tile"``); a request then has
        ``ceil(qo_len * group / 128)`` symbol rows.  ``gqa_symbols="per_q_head"`` instead reads
        symbols per (128-token block, q head), ``bit = q_block * num_qo_heads + q_head`` (no
        counterpart in the reference).  The host planner tiles the batch into the
        integer workspace; in addition the q-block table of the symbol decoder is built and the
        work-list buffers are sized for the worst case (every bit set).  Cannot be captured in a
        graph (it copies the indptrs to the host)."""
        q_data_type = canonicalize_torch_dtype(q_data_type)
        if kv_data_type is None:
            kv_data_type = q_data_type
        kv_data_type = canonicalize_torch_dtype(kv_data_type)
        if head_dim_vo is None:
            head_dim_vo = head_dim_qk
        if logits_soft_cap is None:
            logits_soft_cap = 0.0

        batch_size = len(qo_indptr) - 1
        if len(kv_indptr) != batch_size + 1:
            raise ValueError("The kv_indptr length should be equal to mask_indptr length.")
        _check_pos_encoding_mode(pos_encoding_mode)
        if custom_mask is not None or packed_custom_mask is not None or causal:
            raise NotImplementedError(
                "causal / custom masks are not part of the sparse prefill path (the reference build "
                "only instantiates the non-causal kernel)")
        if PosEncodingMode[pos_encoding_mode] != PosEncodingMode.NONE or use_fp16_qk_reduction:
            raise NotImplementedError(
                "positional encoding and fp16 logits are not part of the sparse prefill path")
        if not (0.0 <= logits_soft_cap < float("inf")):
            raise ValueError("logits_soft_cap must be a finite value >= 0")
        if num_kv_heads <= 0 or num_qo_heads % num_kv_heads != 0:
            raise ValueError("num_qo_heads must be a multiple of num_kv_heads")
        if gqa_symbols not in (None, "packed_tile", "per_q_head"):
            raise ValueError("gqa_symbols must be None, 'packed_tile' or 'per_q_head'")
        if head_dim_qk != 128 or head_dim_vo != 128:
            raise NotImplementedError("only head_dim 128 is supported")
        if sparse_block_size_for_q != 128 or sparse_block_size_for_kv != 128:
            raise NotImplementedError("only 128 x 128 sparse blocks are supported")

        qo_indptr_host = qo_indptr.to("cpu", torch.int32).contiguous()
        kv_indptr_host = kv_indptr.to("cpu", torch.int32).contiguous()
        total_num_rows = int(qo_indptr_host[-1])
        # the attention kernel stages one row's kv block list in LDS (4096 entries)
        if kv_indptr_host.numel() > 1 and int((kv_indptr_host[1:] - kv_indptr_host[:-1]).max()) > 4096 * 128:
            raise NotImplementedError("requests longer than 524288 kv tokens are not supported")

        if self.is_cuda_graph_enabled:
            if self._max_total_num_rows is None:
                self._max_total_num_rows = total_num_rows
            elif total_num_rows > self._max_total_num_rows:
                raise ValueError(
                    "The total number of rows in qo_indptr {} in cuda graph mode cannot "
                    "exceed the number of rows set during initialization {}.".format(
                        total_num_rows, self._max_total_num_rows))
            if batch_size != self._fixed_batch_size:
                raise ValueError(
                    "The batch size should be fixed in cudagraph mode, the runtime batch size {} "
                    " mismatches the batch size set during initialization {}.".format(
                        batch_size, self._fixed_batch_size))
            self._qo_indptr_buf.copy_(qo_indptr)
            self._kv_indptr_buf.copy_(kv_indptr)
        else:
            self._qo_indptr_buf = qo_indptr_host.to(self.device)
            self._kv_indptr_buf = kv_indptr_host.to(self.device)

        self._cached_q_data_type = q_data_type
        self._cached_kv_data_type = kv_data_type

        L = _lib.lib()
        stream = _lib.current_stream(self.device)
        plan_info = torch.empty(15, dtype=torch.int64)
        with torch.cuda.device(self.device):
            try:
                _lib.check(L.fo_prefill_plan(
                    _lib.ptr(self._float_workspace_buffer),
                    self._float_workspace_buffer.numel() * self._float_workspace_buffer.element_size(),
                    _lib.ptr(self._int_workspace_buffer),
                    _lib.ptr(self._pin_memory_int_workspace_buffer),
                    self._int_workspace_buffer.numel() * self._int_workspace_buffer.element_size(),
                    _lib.ptr(qo_indptr_host), _lib.ptr(kv_indptr_host),
                    self._max_total_num_rows or total_num_rows, batch_size, num_qo_heads,
                    num_kv_heads, head_dim_qk, head_dim_vo, 1, int(self.is_cuda_graph_enabled),
                    q_data_type.itemsize, 0, _lib.ptr(plan_info), stream))
            except RuntimeError as e:  # same wording as csrc/batch_sparseFA.cu:61
                raise RuntimeError("Failed to plan prefill with error: " + str(e)) from None
        self._plan_info = plan_info

        self._planned = PlannedBatch(
            self._float_workspace_buffer, qo_indptr_host, kv_indptr_host, self._qo_indptr_buf,
            self._kv_indptr_buf, num_qo_heads, num_kv_heads, sparse_block_size_for_q,
            sparse_block_size_for_kv, share_rows=self._share_rows,
            worklist=self._planned.worklist if self._planned is not None else None,
            gqa_packed=gqa_symbols != "per_q_head")

        self._num_qo_heads = num_qo_heads
        self._num_kv_heads = num_kv_heads
        self._sparse_block_size_for_q = sparse_block_size_for_q
        self._sparse_block_size_for_kv = sparse_block_size_for_kv
        self._causal = causal
        self._pos_encoding_mode = pos_encoding_mode
        self._use_fp16_qk_reduction = use_fp16_qk_reduction
        self._logits_soft_cap = logits_soft_cap
        self._sm_scale = sm_scale
        self._rope_scale = rope_scale
        self._rope_theta = rope_theta

        self._sparse_info_indptr_base = _compute_sparse_info_indptr(
            self._qo_indptr_buf, num_qo_heads, self._sparse_block_size_for_q, device=self.device)
        self._sparse_kv_info_indptr_base = _compute_sparse_kv_info_indptr(
            self._qo_indptr_buf, self._kv_indptr_buf, num_qo_heads, self._sparse_block_size_for_q,
            self._sparse_block_size_for_kv, device=self.device)

    begin_forward = plan

    # names kept for callers that inspect the wrapper
    @property
    def _worklist(self):
        return None if self._planned is None else self._planned.worklist

    @property
    def _split_ok(self):
        return self._planned is not None and self._planned.split_ok

    # ------------------------------------------------------------------------------------------
    def decode(self, sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr,
               is_full: bool = False) -> DecodedWorkList:
        """Decode the packed symbols into the wrapper's work list (asynchronous, on the current
        stream) and return it.  ``run`` calls this itself on every call; a caller that knows the
        symbols have not changed can call it once and then pass ``reuse_decoded=True`` to ``run``."""
        if self._plan_info is None:
            raise RuntimeError("plan() must be called before decode()/run()")
        return self._planned.decode(sparse_info, sparse_kv_info, sparse_info_indptr,
                                    sparse_kv_info_indptr, is_full)

    def run(
        self,
        q: torch.Tensor,
        k: torch.Tensor,
        v: torch.Tensor,
        sparse_info: torch.Tensor = None,
        sparse_kv_info: torch.Tensor = None,
        sparse_info_indptr: torch.Tensor = None,
        sparse_kv_info_indptr: torch.Tensor = None,
        is_full: bool = False,
        *args,
        out: Optional[torch.Tensor] = None,
        lse: Optional[torch.Tensor] = None,
        return_lse: bool = False,
        q_scale: Optional[torch.Tensor] = None,
        k_scale: Optional[torch.Tensor] = None,
        q_lo: Optional[torch.Tensor] = None,
        k_lo: Optional[torch.Tensor] = None,
        reuse_decoded: bool = False,
    ) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
        r"""Compute block-sparse prefill attention.

        q ``[qo_indptr[-1], H, D]``, k/v ``[kv_indptr[-1], H, D]`` (``NHD``) or ``[H, nnz, D]``
        (``HND``).  Rows of q-blocks whose ``sparse_info`` bit is 0 are left untouched in ``out``
        (a fresh ``out`` is zero-filled, as in the reference).  Returns ``out`` or ``(out, lse)``
        with the base-2 log-sum-exp ``[nnz_q, H]``.

        ``q_scale`` / ``k_scale`` (keyword-only extension): fp32 ``[H, n_blocks]`` dequantisation
        scales; with them ``q`` and ``k`` are fp8 e4m3fn, ``v`` and ``out`` are bfloat16.
        ``q_lo``: optional second fp8 term of ``q`` (the rounding residual that
        ``quant_fp8_block(..., residual=True)`` / ``flashomni_gemm(..., quant_out="residual")``
        return): the logits are computed from ``q + q_lo``, which leaves only the rounding of ``k``
        in them and brings the output within relative L2 3e-2 of the unquantised result for
        unit-variance q (two e4m3 operands alone give ~3.9e-2).  ``k_lo`` (needs ``q_lo``): the
        same for ``k`` (``quant_fp8_block(k, ..., residual=True)``); the logits then are
        ``k.q + k.q_lo + k_lo.q`` under the same scales, as accurate as 16-bit logits, for data
        on which one e4m3 byte per element of ``k`` is too coarse (q with rms well above 1).

        ``reuse_decoded`` (keyword-only extension): the symbols are decoded on every call, because
        a buffer rewritten in place (by a kernel of the caller's, through the C ABI, ...) looks the
        same from here.  Pass True to skip the decode and run the work list of the previous
        ``decode``/``run``: the caller then vouches that the four symbol tensors have not changed.
        """
        if self._plan_info is None:
            raise RuntimeError("plan() must be called before run()")
        if q.dim() != 3 or v.dim() != 3:
            raise ValueError("q, k and v must be 3-dimensional with head_dim 128")
        _check_cached_qkv_data_type(q, k, self._cached_q_data_type, self._cached_kv_data_type)
        sm_scale = self._sm_scale
        if sm_scale is None:
            sm_scale = 1.0 / math.sqrt(q.size(-1))
        out_dtype = torch.bfloat16 if is_float8(q) else q.dtype
        if return_lse:
            if lse is None:
                lse = torch.empty((q.size(0), q.size(1)), dtype=torch.float32, device=q.device)
            else:
                _check_shape_dtype_device(lse, (q.size(0), q.size(1)), torch.float32, q.device, "lse")
        if out is None:
            out = torch.zeros(q.shape[:-1] + v.shape[-1:], dtype=out_dtype, device=q.device)
        else:
            _check_shape_dtype_device(out, q.shape[:-1] + v.shape[-1:], out_dtype, q.device, "out")
        pb = self._planned
        if reuse_decoded:
            pb.reuse_decoded(is_full)
        else:
            pb.decode(sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr, is_full)
        pb.launch(q, k, v, out, lse if return_lse else None, self._kv_layout, sm_scale, q_scale, k_scale, q_lo,
                  k_lo, logits_soft_cap=self._logits_soft_cap or 0.0)
        return (out, lse) if return_lse else out

    run_return_lse = functools.partialmethod(run, return_lse=True)

    def forward(self, q, k, v, sparse_info=None, sparse_kv_info=None, sparse_info_indptr=None,
                sparse_kv_info_indptr=None, is_full=False, causal=False, pos_encoding_mode="NONE",
                use_fp16_qk_reduction=False, logits_soft_cap=None, sm_scale=None, rope_scale=None,
                rope_theta=None) -> torch.Tensor:
        r"""Warning: This function is deprecated, please use :meth:`run` instead."""
        self._set_forward_options(causal, pos_encoding_mode, use_fp16_qk_reduction, logits_soft_cap,
                                  sm_scale, rope_scale, rope_theta)
        return self.run(q, k, v, sparse_info, sparse_kv_info, sparse_info_indptr,
                        sparse_kv_info_indptr, is_full)

    def forward_return_lse(self, q, k, v, sparse_info=None, sparse_kv_info=None,
                           sparse_info_indptr=None, sparse_kv_info_indptr=None, is_full=False,
                           causal=False, pos_encoding_mode="NONE", use_fp16_qk_reduction=False,
                           logits_soft_cap=None, sm_scale=None, rope_scale=None,
                           rope_theta=None) -> Tuple[torch.Tensor, torch.Tensor]:
        r"""Warning: This function is deprecated, please use :meth:`run_return_lse` instead."""
        self._set_forward_options(causal, pos_encoding_mode, use_fp16_qk_reduction, logits_soft_cap,
                                  sm_scale, rope_scale, rope_theta)
        return self.run_return_lse(q, k, v, sparse_info, sparse_kv_info, sparse_info_indptr,
                                   sparse_kv_info_indptr, is_full)

    def _set_forward_options(self, causal, pos_encoding_mode, use_fp16_qk_reduction,
                             logits_soft_cap, sm_scale, rope_scale, rope_theta):
        if causal or pos_encoding_mode != "NONE" or use_fp16_qk_reduction:
            raise NotImplementedError("only non-causal attention without positional encoding is supported")
        if not (0.0 <= (logits_soft_cap or 0.0) < float("inf")):
            raise ValueError("logits_soft_cap must be a finite value >= 0")
        self._logits_soft_cap = logits_soft_cap or 0.0
        self._sm_scale = sm_scale
        self._rope_scale = rope_scale
        self._rope_theta = rope_theta

    def end_forward(self) -> None:
        r"""Warning: this function is deprecated and has no effect."""
        pass
