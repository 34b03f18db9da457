// Host-side planning: q/kv tiling of a ragged batch into the caller's integer workspace, and the
// q-block table the sparse-symbol decoder walks.  Pure CPU arithmetic plus one H2D copy.
//
// Behaviour follows the reference planner (include/flashomni/attention/scheduler.cuh:35-168,
// 248-349): q tile size from the average packed q length, the smallest kv chunk (>= 128) whose
// tile count fits 2*CUs/num_kv_heads, tiles enumerated request-major / q-tile-major /
// kv-tile-minor, arrays laid out at 16-byte aligned offsets of the integer workspace.
#include <algorithm>
#include <cstring>
#include <vector>

#include "fo_common.h"

namespace {

struct Bump {
  size_t cur = 0, size = 0;
  bool ok = true;
  explicit Bump(size_t s) : size(s) {}
  int64_t alloc(size_t bytes, size_t align) {
    size_t start = (cur + align - 1) / align * align;
    if (start + bytes > size) {
      ok = false;
      return 0;
    }
    cur = start + bytes;
    return static_cast<int64_t>(start);
  }
};

uint32_t cta_tile_q_for(int64_t avg_packed_qo_len, uint32_t head_dim) {
  if (avg_packed_qo_len > 64 && head_dim < 256) return 128;
  return avg_packed_qo_len > 16 ? 64 : 16;
}

}  // namespace

extern "C" int fo_prefill_plan(void* float_ws, size_t float_ws_bytes, void* int_ws_dev,
                               void* int_ws_host, size_t int_ws_bytes,
                               const int32_t* qo_indptr, const int32_t* kv_indptr,
                               uint32_t total_num_rows, uint32_t batch_size,
                               uint32_t num_qo_heads, uint32_t num_kv_heads, uint32_t head_dim_qk,
                               uint32_t head_dim_vo, uint32_t page_size, int enable_graph,
                               uint32_t sizeof_dtype_o, int num_cu, int64_t plan_info[15],
                               void* stream) {
  (void)float_ws;
  (void)head_dim_qk;
  (void)sizeof_dtype_o;
  FO_REQUIRE(qo_indptr && kv_indptr && int_ws_host && plan_info, "plan: null pointer");
  FO_REQUIRE(batch_size > 0, "plan: batch_size must be positive");
  FO_REQUIRE(num_kv_heads > 0 && num_qo_heads % num_kv_heads == 0,
             "num_qo_heads %u should be divisible by num_kv_heads %u", num_qo_heads, num_kv_heads);
  FO_REQUIRE(page_size > 0, "plan: page_size must be positive");
  if (num_cu <= 0) num_cu = fo_num_cu();
  FO_REQUIRE(num_cu > 0, "plan: no device and no compute-unit count given");

  const int64_t group = num_qo_heads / num_kv_heads;
  std::vector<int64_t> packed(batch_size), kvl(batch_size);
  for (uint32_t i = 0; i < batch_size; ++i) {
    packed[i] = int64_t(qo_indptr[i + 1] - qo_indptr[i]) * group;
    FO_REQUIRE(packed[i] >= 0, "qo_indptr[%u]%d - qo_indptr[%u]%d should be non-negative", i + 1,
               qo_indptr[i + 1], i, qo_indptr[i]);
    kvl[i] = int64_t(kv_indptr[i + 1] - kv_indptr[i]);
    FO_REQUIRE(kvl[i] >= 0, "kv_indptr[%u]%d - kv_indptr[%u]%d should be non-negative", i + 1,
               kv_indptr[i + 1], i, kv_indptr[i]);
  }

  const int64_t max_batch_if_split = (2 * int64_t(num_cu)) / num_kv_heads;
  const int64_t min_kv_chunk = std::max<int64_t>(128 / page_size, 1);
  uint32_t cta_tile_q;
  int64_t total_tiles_q = 0;
  if (enable_graph) {
    const int64_t max_seq = int64_t(total_num_rows) - batch_size + 1;
    cta_tile_q = cta_tile_q_for(max_seq * group, head_dim_vo);
    total_tiles_q = fo::ceil_div(int64_t(total_num_rows) * group, cta_tile_q) + batch_size - 1;
  } else {
    int64_t sum = 0;
    for (int64_t p : packed) sum += p;
    cta_tile_q = cta_tile_q_for(sum / batch_size, head_dim_vo);
    for (int64_t p : packed) total_tiles_q += fo::ceil_div(p, cta_tile_q);
  }

  // smallest kv chunk whose tile count fits
  int64_t max_kv_len = 1;
  for (int64_t x : kvl) max_kv_len = std::max(max_kv_len, x);
  int64_t low = min_kv_chunk, high = max_kv_len;
  while (low < high) {
    const int64_t mid = (low + high) / 2;
    int64_t nb = 0;
    for (uint32_t i = 0; i < batch_size; ++i)
      nb += int64_t(fo::ceil_div(packed[i], cta_tile_q)) *
            fo::ceil_div(std::max<int64_t>(kvl[i], 1), mid);
    if (nb > max_batch_if_split) {
      low = mid + 1;
    } else {
      high = mid;
    }
  }
  const bool split_kv = enable_graph || low < max_kv_len;
  int64_t kv_chunk = low;

  std::vector<int32_t> req, qt, kt, o_indptr(1, 0), merge(1, 0);
  for (uint32_t r = 0; r < batch_size; ++r) {
    const int64_t ntq = fo::ceil_div(packed[r], cta_tile_q);
    const int64_t ntk = fo::ceil_div(std::max<int64_t>(kvl[r], 1), kv_chunk);
    for (int64_t a = 0; a < ntq; ++a)
      for (int64_t b = 0; b < ntk; ++b) {
        req.push_back(int32_t(r));
        qt.push_back(int32_t(a));
        kt.push_back(int32_t(b));
      }
    const int64_t qo_len = packed[r] / group;
    if (split_kv)
      for (int64_t row = 0; row < qo_len; ++row) merge.push_back(int32_t(merge.back() + ntk));
    o_indptr.push_back(int32_t(o_indptr.back() + qo_len * ntk));
  }
  const int64_t new_batch = int64_t(req.size());
  const int64_t padded =
      enable_graph ? std::max<int64_t>(max_batch_if_split, total_tiles_q) : new_batch;
  FO_REQUIRE(new_batch <= padded, "new batch size should not exceed padded batch size");
  kv_chunk *= page_size;

  Bump ib(int_ws_bytes);
  const int64_t off_req = ib.alloc(4 * padded, 16);
  const int64_t off_qt = ib.alloc(4 * padded, 16);
  const int64_t off_kt = ib.alloc(4 * padded, 16);
  const int64_t off_o = ib.alloc(4 * (size_t(batch_size) + 1), 16);
  const int64_t off_chunk = ib.alloc(4, 1);
  int64_t off_rows = 0, off_merge = 0, off_valid = 0, off_v = 0, off_s = 0;
  if (enable_graph) off_rows = ib.alloc(4, 16);
  if (split_kv) {
    Bump fb(float_ws_bytes);
    off_v = fb.alloc(size_t(num_qo_heads) * padded * cta_tile_q * head_dim_vo * sizeof(float), 16);
    off_s = fb.alloc(size_t(num_qo_heads) * padded * cta_tile_q * sizeof(float), 16);
    if (!fb.ok)
      return fo::fail(FO_ERR_WORKSPACE,
                      "Failed to allocate memory for batch_prefill_tmp_v/s in the float workspace "
                      "(%zu bytes)", float_ws_bytes);
    off_merge = ib.alloc(4 * (size_t(total_num_rows) + 1), 16);
    off_valid = ib.alloc(size_t(padded), 16);
  }
  if (!ib.ok)
    return fo::fail(FO_ERR_WORKSPACE,
                    "Failed to allocate memory for the prefill plan in the integer workspace "
                    "(%zu bytes)", int_ws_bytes);

  char* h = static_cast<char*>(int_ws_host);
  std::memcpy(h + off_req, req.data(), 4 * req.size());
  std::memcpy(h + off_qt, qt.data(), 4 * qt.size());
  std::memcpy(h + off_kt, kt.data(), 4 * kt.size());
  std::memcpy(h + off_o, o_indptr.data(), 4 * o_indptr.size());
  const int32_t chunk32 = int32_t(kv_chunk);
  std::memcpy(h + off_chunk, &chunk32, 4);
  if (enable_graph) {
    const uint32_t rows = uint32_t(qo_indptr[batch_size]);
    std::memcpy(h + off_rows, &rows, 4);
  }
  if (split_kv) {
    std::memcpy(h + off_merge, merge.data(), 4 * merge.size());
    for (int64_t i = 0; i < padded; ++i) h[off_valid + i] = i < new_batch;
  }

  const int64_t info[15] = {padded,   total_num_rows, off_rows, cta_tile_q, off_req,
                            off_qt,   off_kt,         off_merge, off_o,     off_chunk,
                            off_v,    off_s,          off_valid, enable_graph ? 1 : 0,
                            split_kv ? 1 : 0};
  std::memcpy(plan_info, info, sizeof(info));

  if (int_ws_dev) {
    FO_HIP_CALL(hipMemcpyAsync(int_ws_dev, int_ws_host, ib.cur, hipMemcpyHostToDevice,
                               static_cast<hipStream_t>(stream)));
  }
  return FO_OK;
}

extern "C" int fo_sparse_block_table(const int32_t* qo_indptr, uint32_t batch_size,
                                     uint32_t block_q, int32_t* blk_req, int32_t* blk_qb,
                                     int64_t capacity, int64_t* n_blk_out) {
  FO_REQUIRE(qo_indptr && n_blk_out && block_q > 0, "block table: bad argument");
  int64_t n = 0;
  for (uint32_t r = 0; r < batch_size; ++r) {
    const int64_t len = int64_t(qo_indptr[r + 1]) - qo_indptr[r];
    FO_REQUIRE(len >= 0, "qo_indptr should be non-decreasing");
    const int64_t nq = (len + block_q - 1) / block_q;
    for (int64_t b = 0; b < nq; ++b, ++n) {
      if (blk_req && blk_qb) {
        if (n >= capacity)
          return fo::fail(FO_ERR_WORKSPACE, "block table: capacity %lld too small",
                          static_cast<long long>(capacity));
        blk_req[n] = int32_t(r);
        blk_qb[n] = int32_t(b);
      }
    }
  }
  *n_blk_out = n;
  return FO_OK;
}

extern "C" int fo_decode_sizes(const int32_t* qo_indptr, const int32_t* kv_indptr,
                               uint32_t batch_size, uint32_t num_heads, uint32_t block_q,
                               uint32_t block_kv, int64_t* n_blk_out, int64_t* max_rows_out,
                               int64_t* max_nnz_out) {
  FO_REQUIRE(qo_indptr && kv_indptr && block_q > 0 && block_kv > 0, "decode sizes: bad argument");
  int64_t n_blk = 0, nnz = 0;
  for (uint32_t r = 0; r < batch_size; ++r) {
    const int64_t ql = int64_t(qo_indptr[r + 1]) - qo_indptr[r];
    const int64_t kl = int64_t(kv_indptr[r + 1]) - kv_indptr[r];
    FO_REQUIRE(ql >= 0 && kl >= 0, "indptr should be non-decreasing");
    const int64_t nq = (ql + block_q - 1) / block_q, nk = (kl + block_kv - 1) / block_kv;
    n_blk += nq;
    nnz += nq * nk * num_heads;
  }
  if (n_blk_out) *n_blk_out = n_blk;
  if (max_rows_out) *max_rows_out = n_blk * num_heads;
  if (max_nnz_out) *max_nnz_out = nnz;
  return FO_OK;
}
