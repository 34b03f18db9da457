/*
 * flashomni_hip.h -- C ABI of the MI355X (gfx950) FlashOmni sparse-attention engine.
 *
 * Plain pointers and sizes only; no torch types.  Every entry point that touches the GPU
 * takes the HIP stream to enqueue on (a hipStream_t passed as void*; NULL = the null stream),
 * never synchronises and never allocates device memory.  Return value: 0 on success, a
 * negative FO_ERR_* code otherwise; fo_last_error() then holds a thread-local message.
 *
 * Each entry point names the reference interface it stands in for (paths are relative to the
 * root of qiaolian9/FlashOmni).
 */
#ifndef FLASHOMNI_HIP_H_
#define FLASHOMNI_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FO_ABI_VERSION 5

enum {
  FO_OK = 0,
  FO_ERR_INVALID = -1,   /* bad argument / unsupported shape (reference: TORCH_CHECK failures) */
  FO_ERR_WORKSPACE = -2, /* workspace too small (reference: AlignedAllocator overflow) */
  FO_ERR_HIP = -3        /* a HIP runtime call failed (reference: cudaError_t return codes) */
};

/* element types of activations */
enum { FO_BF16 = 0, FO_F16 = 1, FO_FP8_E4M3 = 2, FO_F32 = 3 };
/* bit orders of packbits */
enum { FO_BITORDER_BIG = 0, FO_BITORDER_LITTLE = 1 };
/* kinds of the GEMM-O `bias` operand */
enum { FO_BIAS_NONE = 0, FO_BIAS_VECTOR = 1, FO_BIAS_MATRIX = 2 };

const char* fo_last_error(void);
int fo_abi_version(void);
/* number of compute units of the current device (0 if no device) */
int fo_num_cu(void);

/* ---------------------------------------------------------------------------------------------
 * packbits / segment_packbits
 * replaces: csrc/quantization.cu:22-36 (packbits), :38-57 (segment_packbits);
 *           kernels include/flashomni/quantization.cuh:39-57, :59-83.
 * x: n bool bytes (non-zero = 1) on the device; y: ceil(n/8) bytes.
 * segment form: indptrs are int32 device arrays of num_segments+1 entries; segment i packs
 * x[in_indptr[i] : in_indptr[i+1]] into y[out_indptr[i] : ...], starting on a byte boundary.
 * ------------------------------------------------------------------------------------------- */
int fo_packbits(const uint8_t* x, int64_t n, int bitorder, uint8_t* y, void* stream);
int fo_segment_packbits(const uint8_t* x, const int32_t* in_indptr, const int32_t* out_indptr,
                        int32_t num_segments, int bitorder, uint8_t* y, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Host planner.
 * replaces: BatchSparseFAWithKVPlan csrc/batch_sparseFA.cu:39-65 and PrefillPlan
 *           include/flashomni/attention/scheduler.cuh:248-349 (+ :35-168, utils.cuh:293-312,
 *           allocator.h:32-58).
 * Pure host arithmetic: fills the pinned mirror `int_ws_host` with request_indices,
 * qo_tile_indices, kv_tile_indices, o_indptr, kv_chunk_size (and merge_indptr,
 * block_valid_mask when kv is split) at 16-byte aligned offsets and writes the 15-entry plan
 * vector in the reference's order (scheduler.cuh:205-221).  When int_ws_dev is not NULL the
 * used prefix is copied host->device on `stream`.  num_cu <= 0 queries the current device.
 * ------------------------------------------------------------------------------------------- */
int fo_prefill_plan(void* float_ws, size_t float_ws_bytes, void* int_ws_dev, void* int_ws_host,
                    size_t int_ws_bytes, const int32_t* qo_indptr_host,
                    const int32_t* kv_indptr_host, uint32_t total_num_rows, uint32_t batch_size,
                    uint32_t num_qo_heads, uint32_t num_kv_heads, uint32_t head_dim_qk,
                    uint32_t head_dim_vo, uint32_t page_size, int enable_graph,
                    uint32_t sizeof_dtype_o, int num_cu, int64_t plan_info_out[15], void* stream);

/* ---------------------------------------------------------------------------------------------
 * Sparse-symbol decoder: packed symbols -> compacted, canonically ordered work list.
 * replaces the per-CTA bit tests and bit walks of
 *   include/flashomni/attention/prefill.cuh:1284-1294 (q-block flag),
 *   :1380-1403 and :1434-1460 (next kept kv block).
 *
 * The q-block table (one entry per sparse q-block of every request, request-major) is built on
 * the host by fo_sparse_block_table(); fo_decode_sizes() tells how large the outputs must be.
 *
 * Bit conventions: bit = 1 keep/compute; little-endian in a byte; sparse_info bit index inside
 * request r is qb*H + h; sparse_kv_info bit index is (qb*H + h)*NKV_r + kvb with
 * NKV_r = ceil(kv_len_r / block_kv); the two indptr arrays are BYTE offsets per request.
 *
 * Outputs (all int32, device):
 *   row_req,row_qb,row_head [n_rows]  rows with flag 1, ascending (request, q-block, head)
 *   kv_row_ptr [n_rows+1], kv_idx [nnz]  kept kv blocks of each row, ascending
 *   counts[0] = n_rows, counts[1] = nnz, counts[2..3] = 0
 *   order [n_rows]   execution order for the attention kernel: canonical row positions grouped by
 *                    head, heads dealt round-robin to 8 queues (head % 8, one queue per XCD).  Inside
 *                    one head: with eight or more rows per CU, ascending (request, q block), a fixed
 *                    order in which the entries popped together share kv blocks (sched[32] = 1);
 *                    with fewer, longer rows first (up to 32 length classes), otherwise unspecified
 *   sched [1024]     sched[0..8] = queue boundaries inside `order`, sched[16..23] = queue cursors
 *                    and sched[24] = completion counter, both cleared to 0; sched[25] = kv count of
 *                    the longest row; sched[26..30] = even shares: in use, cost share of a
 *                    workgroup, total cost, number of shares, number of rows; sched[31] = the
 *                    share table holds queue-entry records; sched[32] = `order` is the fixed
 *                    ascending one;
 *                    sched[64..575] = arrival counters of rows cut at share boundaries (cleared)
 * shares (optional, [512 + 8*(n_blk*H + 1)] int32, 16-byte aligned): scheduling table for the
 * attention kernel, to be passed to fo_sparse_fa_run with the list.  Normally (sched[31] = 1) it
 * receives one 8-int record per entry of `order`, at shares[512 + 8*i]: row, request, q block,
 * head, first kv_idx slot, kv block count, 0, 0, so that a popped entry costs the attention kernel
 * one load instead of three dependent rounds.  When the list holds at most 2 rows per CU the
 * decoder lays out even shares instead (sched[26] = 1): `order` then lists the rows head by head
 * (q blocks ascending: a fixed order), a row costs 3 + its kv blocks, shares[512 + i] is the cost
 * at which the kv blocks of row order[i] begin, share j is the cost range
 * [j*sched[27], (j+1)*sched[27]) and shares[j] its first row.  The attention kernel gives every
 * workgroup one share and computes a row that straddles a boundary in parts (consecutive ranges
 * of its kv blocks, at most 4), one per share it touches (the counterpart of the reference's
 * split-kv plan, scheduler.cuh:35-64, decided on the device from the decoded list).  The queues
 * stay valid (eight equal runs of `order`), and the canonical lists do not change.
 * is_full != 0 ignores the symbol tensors (which may be NULL) and lists everything
 * (csrc/batch_sparseFA.cu:123-128).
 * `scratch` needs 2*n_blk*H + 8192 int32.
 * ------------------------------------------------------------------------------------------- */
int fo_sparse_block_table(const int32_t* qo_indptr_host, uint32_t batch_size, uint32_t block_q,
                          int32_t* blk_req_host, int32_t* blk_qb_host, int64_t capacity,
                          int64_t* n_blk_out);
int fo_decode_sizes(const int32_t* qo_indptr_host, const int32_t* kv_indptr_host,
                    uint32_t batch_size, uint32_t num_heads, uint32_t block_q, uint32_t block_kv,
                    int64_t* n_blk_out, int64_t* max_rows_out, int64_t* max_nnz_out);
int fo_decode_sparse(const uint8_t* sparse_info, const uint8_t* sparse_kv_info,
                     const int32_t* sparse_info_indptr, const int32_t* sparse_kv_info_indptr,
                     const int32_t* blk_req, const int32_t* blk_qb, const int32_t* kv_indptr,
                     int32_t n_blk, int32_t num_heads, int32_t block_kv, int is_full,
                     int32_t* row_req, int32_t* row_qb, int32_t* row_head, int32_t* kv_row_ptr,
                     int32_t* kv_idx, int32_t* counts, int32_t* order, int32_t* sched,
                     int32_t* scratch, int32_t* shares, void* stream);

/* ---------------------------------------------------------------------------------------------
 * fo_decode_sparse without the `scratch` argument, for callers that cannot allocate device memory
 * for it (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * No counterpart in the reference.  The decoder's scratch (2*n_blk*H + 8192 int32) lives in a 1 MiB
 * array built into the library's device code instead (one copy per GPU, held until the process ends),
 * so n_blk * num_heads may be at most fo_decode_sparse_static_max_pairs() (126 976); larger
 * inputs are refused with FO_ERR_INVALID.  Same inputs, outputs and results as fo_decode_sparse.
 * The call allocates nothing.  Its first call on a device looks up the array's address, which is not
 * a stream operation: make one call on every device outside any capture (any small input will do)
 * before capturing the entry point into a graph; later calls only launch kernels.  All calls
 * on one GPU share that array: calls that overlap in time on one GPU (two streams, two threads)
 * race; calls on one stream are safe.
 * ------------------------------------------------------------------------------------------- */
int64_t fo_decode_sparse_static_max_pairs(void);
int fo_decode_sparse_static(const uint8_t* sparse_info, const uint8_t* sparse_kv_info,
                            const int32_t* sparse_info_indptr, const int32_t* sparse_kv_info_indptr,
                            const int32_t* blk_req, const int32_t* blk_qb, const int32_t* kv_indptr,
                            int32_t n_blk, int32_t num_heads, int32_t block_kv, int is_full,
                            int32_t* row_req, int32_t* row_qb, int32_t* row_head, int32_t* kv_row_ptr,
                            int32_t* kv_idx, int32_t* counts, int32_t* order, int32_t* sched,
                            int32_t* shares, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Ragged block-sparse FlashAttention prefill over a decoded work list.
 * replaces: BatchSparseFAWithRaggedKVRun csrc/batch_sparseFA.cu:67-201 and the kernel
 *           include/flashomni/attention/prefill.cuh:1203-1531 (mask none, no positional
 *           encoding, fp32 logits: the only variant the reference builds, setup.py:98-111).
 *
 * q [nnz_q,H,D], k,v [nnz_kv,H_kv,D], o [nnz_q,H,D]; strides in elements (the innermost stride is
 * 1).  num_heads = H must be a multiple of num_kv_heads = H_kv: q head h reads kv head
 * h / (H / H_kv) (grouped-query attention, prefill.cuh:410-413); k_scale then has H_kv rows.
 * gqa_packed selects what a work-list row is when H_kv < H (it has no effect when H_kv = H):
 *   1: the reference's layout (prefill.cuh:1283-1290 with :410-413): a request's q rows are its
 *      (token, q head of the group) pairs, token-major, per kv head; row (request, tile t, kv head j)
 *      covers pairs t*128 .. t*128+127, i.e. pair r is token r / g, q head j*g + r % g (g = H / H_kv),
 *      and the symbols hold one bit per (tile, kv head) (x one per kv block): the list is decoded
 *      with num_heads = H_kv over ceil(qo_len * g / 128) tiles per request, row_qb is the tile and
 *      row_head the kv head.  16-bit q, k, v only.
 *   0: a row is (request, 128-token block, q head), symbols per q head (no reference counterpart).
 * dtype FO_BF16 / FO_F16: q,k,v,o share it.  dtype FO_FP8_E4M3: q and k are e4m3fn bytes
 * with dequantisation scales q_scale[H][n_q_blocks], k_scale[H][n_kv_blocks] (fp32, blocks
 * numbered request by request: q_blk_base / kv_blk_base [batch+1] give each request's first
 * block); v and o are bf16.  q_lo (optional, else NULL): a second e4m3fn tensor laid out like q, the
 * rounding residual of q under the same scale (fo_quant_fp8_block / fo_gemm_q_quant write it);
 * the logits are then K.(q + q_lo)^T, two fp8 products at the cost of one 16-bit one, and only k's
 * rounding error is left in them.  k_lo (optional, else NULL; needs q_lo): the same for k, laid out
 * like k under k's scales; the logits are then k.q^T + k.q_lo^T + k_lo.q^T (the product of the two
 * residuals is left out), as accurate as 16-bit logits at three fp8 products per tile: the
 * accuracy form for data on which one e4m3 byte per element of k is too coarse, not a fast one.
 * A request may hold at most 524 288 kv tokens (4096 kv blocks, the list of one row is staged in
 * LDS), with k_lo 262 144: the caller checks that (the lengths live on the device).
 * (The fp8 form has no counterpart in the reference.)
 * Rows of the list write every output row of their q-block; q-blocks not in the list are left
 * untouched; a listed row with no kv block writes zeros and lse = -5e4.  lse (optional, fp32
 * [nnz_q,H]) is base 2: log2(sum 2^(s*c - m*c)) + m*c, c = sm_scale*log2(e).
 * logits_soft_cap > 0 (16-bit q/k only; 0 = off): the scores become cap * tanh(q.k * sm_scale / cap)
 * before the softmax, and lse is taken over those (reference: DefaultAttention with
 * use_logits_soft_cap, include/flashomni/attention/variants.cuh:43-56, :68-70; tanh is formed as
 * 1 - 2 / (1 + exp(2x)) where the reference uses tanh.approx).  Runs in the 8-wavefront form whatever
 * the list's length.
 * Rows are taken from the queues described by `order` / `sched` (see fo_decode_sparse); the
 * kernel leaves the queue cursors rewound, so one decoded list can be run any number of times,
 * but two launches sharing one `sched` must not overlap in time.
 * shares: the table fo_decode_sparse filled for this list, or NULL.  With it a popped queue entry
 * is read as one record; when the decoder chose even shares every workgroup computes one share; split_workspace, device memory of
 * fo_sparse_fa_split_workspace_bytes() bytes (two areas per CU), 16-byte aligned, is then required
 * and receives the unnormalised partial results (fp32 O, row maximum, row sum) of rows cut at share
 * boundaries: the part that arrives last combines them in part order (replaces the reference's
 * float workspace + merge kernels, scheduler.cuh:322-328, cascade.cuh:346-437).  Without shares
 * the rows are taken whole from the queues.  Launches sharing a workspace must not overlap in time.
 * Supported: D = 128, block_q = 128, block_kv = 128.  max_rows bounds the number of rows.
 * ------------------------------------------------------------------------------------------- */
int64_t fo_sparse_fa_split_workspace_bytes(void);
/* Which form of the kernel fo_sparse_fa_run launches (process-wide; no counterpart in the reference):
 * 0 = automatic (the default): lists whose upper bound max_rows is at least 8 rows per CU run as two
 * independent 4-wavefront workgroups per CU, one row each, with a software-pipelined loop; shorter
 * ones as one 8-wavefront workgroup per CU whose two halves share a row.  1 / 2 force the first /
 * second form where it applies (the first needs 16-bit q, k, v, at most 3072 kv blocks in the batch
 * and kv strides that keep a request's keys within 4 GiB).  Results agree within the stated
 * tolerances, not bit for bit.  For tests and measurements. */
int fo_sparse_fa_set_variant(int variant);
int fo_sparse_fa_run(const void* q, const void* k, const void* v, void* o, float* lse, int dtype,
                     const void* q_lo, const void* k_lo, const float* q_scale, const float* k_scale,
                     int64_t q_stride_n,
                     int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                     int64_t v_stride_n, int64_t v_stride_h, int64_t o_stride_n,
                     int64_t o_stride_h, const int32_t* qo_indptr, const int32_t* kv_indptr,
                     const int32_t* q_blk_base, const int32_t* kv_blk_base, int32_t n_q_blocks,
                     int32_t n_kv_blocks, const int32_t* row_req, const int32_t* row_qb, const int32_t* row_head,
                     const int32_t* kv_row_ptr, const int32_t* kv_idx, const int32_t* order,
                     int32_t* sched, int64_t max_rows, int32_t num_heads, int32_t num_kv_heads, int32_t gqa_packed,
                     int32_t head_dim, int32_t block_q, int32_t block_kv, float sm_scale, float logits_soft_cap,
                     const int32_t* shares, void* split_workspace, int64_t split_workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * GEMM-Q: y[b, tile] = x[b] . w^T + bias for every (128-row, 128-column) tile whose symbol bit
 * is 1; other tiles keep their bytes.
 * replaces: FLASHOMNIGEMM csrc/gemm.cu:24-59, FLASHOMNIGEMMRun/kernel
 *           include/flashomni/gemm/w16a16/gemm.cuh:27-228, :230-357.
 * x [B,M,K], w [N,K], y [B,M,N] row-major contiguous; bias [N] or NULL; dtype FO_BF16/FO_F16.
 * Tile (b, iy, ix) tests bit ((num_text_tokens + iy*128)/sparse_q_size)*num_qo_heads
 * + (ix*128)/(N/num_qo_heads) of sparse_info + sparse_info_indptr[b] (gemm.cuh:50-58).
 * Requires N % 128 == 0, K % 32 == 0 (csrc/gemm.cu:36) and 64 <= K <= 65536; M may have a tail (the
 * reference demands M % 128 == 0).
 * `workspace`: device scratch of at least fo_gemm_workspace_bytes(batch, m, n) bytes, 16-byte
 * aligned; it receives the list of tile quads that the GEMM kernel walks (short launches, up to
 * 256 windows x column pairs, build the list inside the GEMM kernel and leave it untouched).
 * ------------------------------------------------------------------------------------------- */
int64_t fo_gemm_workspace_bytes(int32_t batch, int32_t m, int32_t n);
int fo_gemm_q(const void* x, const void* w, const void* bias, void* y, int dtype, int32_t batch,
              int32_t m, int32_t n, int32_t k, int32_t sparse_q_size, int32_t num_qo_heads,
              const uint8_t* sparse_info, const int32_t* sparse_info_indptr,
              int32_t num_text_tokens, int is_full, void* workspace, int64_t workspace_bytes,
              void* stream);

/* ---------------------------------------------------------------------------------------------
 * GEMM-O with reduction: y[b, row-tile, :] = init + sum over selected head slices of
 * x[:, h*hd:(h+1)*hd] . w[:, h*hd:(h+1)*hd]^T, hd = N/num_qo_heads.
 * is_for_cached != 0 selects heads whose bit is 0 and init = bias vector [N];
 * is_for_cached == 0 selects heads whose bit is 1 and init = bias matrix [B,M,N].
 * replaces: FLASHOMNIGEMMReduction csrc/gemm_reduction.cu:24-57, kernel
 *           include/flashomni/gemm/w16a16/gemm_reduction.cuh:27-276 (:77-95 init, :126-160
 *           slice selection).
 * bias_dtype: the activation dtype (as in the reference) or FO_F32 for the matrix form;
 * y_dtype: the activation dtype or FO_F32 (so a cached partial can stay in fp32).
 * hd must be a multiple of 32.  No tile list is needed (every token block is visited, the tile
 * order is computed arithmetically), so `workspace` may be NULL; fo_gemm_q with is_full != 0
 * likewise.  Given 64 bytes or more of 4-byte-aligned device scratch, a launch with several work
 * items per CU hands them out through cursors kept there (work items of unequal length then stay
 * neighbours in L2); launches that share the scratch must not overlap in time.
 * ------------------------------------------------------------------------------------------- */
int fo_gemm_o(const void* x, const void* w, const void* bias, void* y, int dtype, int bias_kind,
              int bias_dtype, int y_dtype, int32_t batch, int32_t m, int32_t n, int32_t k,
              int32_t sparse_q_size, int32_t num_qo_heads, const uint8_t* sparse_info,
              const int32_t* sparse_info_indptr, int32_t num_text_tokens, int is_for_cached,
              void* workspace, int64_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * GEMM-Q with the fp8 quantisation of its result fused into the epilogue.
 * No counterpart in the reference (it has no fp8 product, see fo_quant_fp8_block); for callers that
 * feed the projection straight into fp8 attention.  As fo_gemm_q, plus: y8 [batch, m, n] e4m3fn
 * bytes and y_scale[num_qo_heads][batch * ceil(m / 128)] fp32, written for the computed tiles only:
 * scale = absmax of the (128-token block, head) slab of the fp32 result (bias included) / 448 (1 for
 * an all-zero slab), y8 = rne(result / scale).  y8_lo (optional, else NULL) [batch, m, n]: the
 * residual rne(result / scale - y8), the second term of a two-term fp8 operand.  y may be NULL (the
 * 16-bit result is then not written).  Needs n / num_qo_heads == 128.
 * ------------------------------------------------------------------------------------------- */
int fo_gemm_q_quant(const void* x, const void* w, const void* bias, void* y, uint8_t* y8,
                    uint8_t* y8_lo, float* y_scale, int dtype, int32_t batch, int32_t m, int32_t n, int32_t k,
                    int32_t sparse_q_size, int32_t num_qo_heads, const uint8_t* sparse_info,
                    const int32_t* sparse_info_indptr, int32_t num_text_tokens, int is_full,
                    void* workspace, int64_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * fp8 e4m3fn quantiser with one absmax scale per (head, 128-token block).
 * No counterpart in the reference (its quantization.cuh only packs bits).
 * x [nnz,H,D] bf16/f16 (strides in elements), x8 [nnz,H,D] bytes contiguous,
 * scale fp32 [H][n_blk]: scale = absmax/448 (1 for an all-zero block), x8 = rne(x/scale).
 * x8_lo (optional, else NULL), laid out like x8: the residual rne(x/scale - x8).
 * blk_req/blk_tok0/blk_len (int32 [n_blk], device): request, first token and length of each block.
 * ------------------------------------------------------------------------------------------- */
int fo_quant_fp8_block(const void* x, int dtype, int64_t x_stride_n, int64_t x_stride_h,
                       uint8_t* x8, uint8_t* x8_lo, float* scale, const int32_t* blk_tok0, const int32_t* blk_len,
                       int32_t n_blk, int32_t num_heads, int32_t head_dim, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Symbol producer: pooled attention scores -> packed sparse_info / sparse_kv_info.
 * replaces: the torch sort / cumsum / searchsorted steps of benchmark/test_attn_score.py:96-105,
 *           :117-127, the Triton fill kernels :5-91, and the transposition + segment_packbits that
 *           turn the maps into run() arguments (benchmark/utils.py:83-84,
 *           benchmark/test_flashomni_attention.py:254-257).
 * scores [batch, H, NQ, NK] contiguous (FO_F32, FO_BF16 or FO_F16), finite.
 * q symbols: the scores of the first n_text_q q blocks towards key blocks n_text_kv.. are summed
 *   over heads and those q blocks and soft-maxed; the key blocks of lowest score whose cumulative
 *   probability stays <= q_threshold[request] are cached: q block n_text_q + j gets symbol 0 for
 *   every head.  kv symbols: each row (head, q block >= n_text_q) is soft-maxed over all NK key
 *   blocks and those of lowest score whose cumulative probability stays <= kv_threshold[head] get
 *   symbol 0; text q rows keep every key block.  Equal scores are taken in index order; cumulative
 *   probabilities are exact sums of probabilities rounded to 2^-30.
 * Outputs (device): sparse_info batch*ceil(NQ*H/8) bytes, sparse_kv_info batch*ceil(NQ*H*NK/8)
 *   bytes, little-endian bits at q_block*H+head resp. (q_block*H+head)*NK+kv_block inside each
 *   request's byte-aligned segment; the two indptr arrays (int32 [batch+1], byte offsets) are
 *   written too.  Every output byte is written: no clearing needed.  NQ, NK <= 4096.
 * ------------------------------------------------------------------------------------------- */
int fo_symbols_from_scores(const void* scores, int dtype, int32_t batch, int32_t num_heads,
                           int32_t n_q_blocks, int32_t n_kv_blocks, int32_t n_text_q,
                           int32_t n_text_kv, const float* q_threshold, const float* kv_threshold,
                           uint8_t* sparse_info, int32_t* sparse_info_indptr,
                           uint8_t* sparse_kv_info, int32_t* sparse_kv_info_indptr, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHOMNI_HIP_H_ */
