// Sparse-symbol decoder for gfx950: bit-packed (head, q-block) flags and (head, q-block, kv-block)
// keep masks -> compacted work list in canonical order (ascending request, q-block, head; kv
// blocks ascending inside a row).  Three short launches on one stream, no host round trip:
//   count : one wavefront per (q-block, head) candidate; lanes take one mask byte each, popcount
//   scan  : one workgroup, exclusive prefix sums of row flags and kv counts (canonical positions),
//           plus a per-head histogram that lays out the execution order
//   fill  : one wavefront per candidate again; wave prefix of popcounts places every kv index
//
// Besides the canonical list the decoder emits an execution order for the attention kernel:
// `order` lists row positions grouped by head, heads dealt to the 8 XCDs round-robin (head % 8), so
// that the workgroups of one XCD (which share an L2) walk the rows of the same few heads and find
// that head's K/V in their L2.  Inside a head the rows go longest first (up to 32 length classes relative
// to the longest row of the launch), which evens out the workgroups' finishing times when there are
// only a few rows per CU.  sched[0..8] delimit the 8 per-XCD queues inside `order`, sched[16..23]
// are the queue cursors, sched[24] a completion counter (all cleared here) and sched[25] the
// longest row's kv count.  sched[32..55] describe, per queue, the rows at its end that the attention
// kernel shares between workgroups, and sched[64..191] are their arrival counters (cleared here).  The order inside a length class is not deterministic (atomic cursors);
// results do not depend on it.
// Integer work, bounded by HBM traffic and launch latency; bit-exact by construction.
//
// Symbol semantics (reference: include/flashomni/attention/prefill.cuh:1284-1294, 1380-1403,
// 1434-1460): bit 1 = compute/keep, little-endian bytes, flag bit index qb*H + h, keep-mask bit
// index (qb*H + h)*NKV + kvb, per-request byte offsets.
#include "fo_common.h"

namespace {

constexpr int kWave = 64;
constexpr int kCountThreads = 256;  // 4 candidates per workgroup
constexpr int kScanThreads = 1024;
constexpr int kMaxHeads = 1024;
constexpr int kXcds = 8;
constexpr int kHistSlots = 8192;  // (head, length class) counters of the order layout
// split rows (see the attention kernel): words of `sched` and limits
constexpr int kSchedSplitStart = 32, kSchedSplitParts = 40, kSchedSplitSlot = 48, kSchedArrived = 64;
constexpr int kMaxSplitSlots = 128, kMaxSplitParts = 4, kSplitMaxRounds = 1;

// number of length classes for num_heads heads (32 up to 256 heads)
__host__ __device__ __forceinline__ int len_classes(int32_t num_heads) {
  const int k = kHistSlots / num_heads;
  return k > 32 ? 32 : k;
}
// length class of a row with n kv blocks when the longest row has max_n: 0 = longest
__device__ __forceinline__ int len_class(int32_t n, int32_t max_n, int n_classes) {
  return static_cast<int>(static_cast<int64_t>(max_n - n) * n_classes / (max_n + 1));
}

struct Candidate {
  int32_t req, qb, head, nkv;
  int64_t base;  // first bit of the row inside the request's keep-mask segment
  bool active;
};

__device__ __forceinline__ Candidate load_candidate(
    int64_t c, int32_t num_heads, int32_t block_kv, int is_full,
    const uint8_t* __restrict__ sparse_info, const int32_t* __restrict__ sparse_info_indptr,
    const int32_t* __restrict__ blk_req, const int32_t* __restrict__ blk_qb,
    const int32_t* __restrict__ kv_indptr) {
  Candidate cd;
  const int64_t t = c / num_heads;
  cd.head = static_cast<int32_t>(c - t * num_heads);
  cd.req = blk_req[t];
  cd.qb = blk_qb[t];
  const int32_t kv_len = kv_indptr[cd.req + 1] - kv_indptr[cd.req];
  cd.nkv = (kv_len + block_kv - 1) / block_kv;
  const int64_t flag_bit = static_cast<int64_t>(cd.qb) * num_heads + cd.head;
  cd.base = flag_bit * cd.nkv;
  if (is_full) {
    cd.active = true;
  } else {
    const uint8_t byte = sparse_info[sparse_info_indptr[cd.req] + (flag_bit >> 3)];
    cd.active = (byte >> (flag_bit & 7)) & 1;
  }
  return cd;
}

// bits of mask byte `b` (absolute byte index inside the segment) that belong to [base, base+nkv)
__device__ __forceinline__ uint32_t masked_byte(const uint8_t* __restrict__ seg, int64_t b,
                                                int64_t base, int32_t nkv) {
  uint32_t v = seg[b];
  const int64_t lo = base - b * 8;             // first valid bit position in this byte
  const int64_t hi = base + nkv - b * 8;       // one past the last valid bit position
  if (lo > 0) v &= 0xffu << lo;
  if (hi < 8) v &= (1u << hi) - 1u;
  return v;
}

__global__ void __launch_bounds__(kCountThreads) decode_count_kernel(
    const uint8_t* __restrict__ sparse_info, const uint8_t* __restrict__ sparse_kv_info,
    const int32_t* __restrict__ sparse_info_indptr,
    const int32_t* __restrict__ sparse_kv_info_indptr, const int32_t* __restrict__ blk_req,
    const int32_t* __restrict__ blk_qb, const int32_t* __restrict__ kv_indptr, int64_t n_cand,
    int32_t num_heads, int32_t block_kv, int is_full, int32_t* __restrict__ act,
    int32_t* __restrict__ cnt) {
  const int lane = threadIdx.x % kWave;
  const int64_t c = static_cast<int64_t>(blockIdx.x) * (kCountThreads / kWave) + threadIdx.x / kWave;
  if (c >= n_cand) return;
  const Candidate cd = load_candidate(c, num_heads, block_kv, is_full, sparse_info,
                                      sparse_info_indptr, blk_req, blk_qb, kv_indptr);
  int32_t total = 0;
  if (cd.active) {
    if (is_full) {
      total = cd.nkv;
    } else if (cd.nkv > 0) {
      const uint8_t* seg = sparse_kv_info + sparse_kv_info_indptr[cd.req];
      const int64_t b0 = cd.base >> 3, b1 = (cd.base + cd.nkv - 1) >> 3;
      int32_t part = 0;
      for (int64_t b = b0 + lane; b <= b1; b += kWave) part += __popc(masked_byte(seg, b, cd.base, cd.nkv));
      for (int off = kWave / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, kWave);
      total = part;
    }
  }
  if (lane == 0) {
    act[c] = cd.active ? 1 : 0;
    cnt[c] = total;
  }
}

// In place: act[c] -> canonical row position (or -1), cnt[c] -> first kv_idx slot of the row.
__global__ void __launch_bounds__(kScanThreads) decode_scan_kernel(
    int64_t n_cand, int32_t num_heads, int32_t* __restrict__ act, int32_t* __restrict__ cnt,
    int32_t* __restrict__ kv_row_ptr, int32_t* __restrict__ counts,
    int32_t* __restrict__ head_cursor, int32_t* __restrict__ sched, int32_t cus_per_xcd) {
  __shared__ int32_t s_rows[kScanThreads];
  __shared__ int32_t s_kv[kScanThreads];
  __shared__ int32_t s_hist[kHistSlots];
  __shared__ int32_t s_max;
  const int tid = threadIdx.x;
  const int n_classes = len_classes(num_heads);
  for (int h = tid; h < num_heads * n_classes; h += kScanThreads) s_hist[h] = 0;
  if (tid == 0) s_max = 0;
  __syncthreads();
  const int64_t chunk = (n_cand + kScanThreads - 1) / kScanThreads;
  const int64_t lo = tid * chunk, hi = (lo + chunk < n_cand) ? lo + chunk : n_cand;
  int32_t rows = 0, kv = 0, mx = 0;
  for (int64_t c = lo; c < hi; ++c) {
    rows += act[c];
    kv += cnt[c];
    mx = max(mx, cnt[c]);
  }
  atomicMax(&s_max, mx);
  __syncthreads();
  const int32_t max_n = s_max;
  for (int64_t c = lo; c < hi; ++c)
    if (act[c]) atomicAdd(&s_hist[(c % num_heads) * n_classes + len_class(cnt[c], max_n, n_classes)], 1);
  s_rows[tid] = rows;
  s_kv[tid] = kv;
  __syncthreads();
  // Hillis-Steele inclusive scan over the 1024 partials
  for (int off = 1; off < kScanThreads; off <<= 1) {
    int32_t r = 0, k = 0;
    if (tid >= off) {
      r = s_rows[tid - off];
      k = s_kv[tid - off];
    }
    __syncthreads();
    s_rows[tid] += r;
    s_kv[tid] += k;
    __syncthreads();
  }
  int32_t row_pos = s_rows[tid] - rows, kv_pos = s_kv[tid] - kv;
  for (int64_t c = lo; c < hi; ++c) {
    const int32_t a = act[c], n = cnt[c];
    act[c] = a ? row_pos : -1;
    cnt[c] = kv_pos;
    row_pos += a;
    kv_pos += n;
  }
  if (tid == kScanThreads - 1) {
    const int32_t n_rows = s_rows[tid], nnz = s_kv[tid];
    counts[0] = n_rows;
    counts[1] = nnz;
    counts[2] = 0;
    counts[3] = 0;
    kv_row_ptr[n_rows] = nnz;
  }
  // execution order layout: queue x holds heads x, x+8, x+16, ... back to back, each head's length
  // classes in order.  Exclusive prefix sum of the histogram taken in that order: every thread owns
  // a run of consecutive entries, wavefront scan by lane shifts, then the sixteen wavefront totals.
  __syncthreads();  // s_rows / s_kv are free again
  {
    const int n_ent = num_heads * n_classes;
    const int per = (n_ent + kScanThreads - 1) / kScanThreads;
    const int e_lo = min(tid * per, n_ent), e_hi = min(e_lo + per, n_ent);
    // entry j of the order -> slot of the histogram: j / n_classes is the head's rank in queue order
    auto slot_of = [&](int j, int* queue) {
      const int rank = j / n_classes, k = j - rank * n_classes;
      int x = 0, base = 0;
      for (; x < kXcds; ++x) {
        const int c = num_heads > x ? (num_heads - x + kXcds - 1) / kXcds : 0;  // heads of queue x
        if (rank < base + c) break;
        base += c;
      }
      *queue = x;
      return (x + kXcds * (rank - base)) * n_classes + k;
    };
    int32_t mine = 0;
    int qx;
    for (int j = e_lo; j < e_hi; ++j) mine += s_hist[slot_of(j, &qx)];
    const int lane = tid & 63, wave = tid >> 6;
    int32_t incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int32_t up = __shfl_up(incl, d, 64);
      if (lane >= d) incl += up;
    }
    if (lane == 63) s_rows[wave] = incl;
    __syncthreads();
    int32_t pos = incl - mine;
    for (int w = 0; w < wave; ++w) pos += s_rows[w];
    for (int j = e_lo; j < e_hi; ++j) {
      const int slot = slot_of(j, &qx);
      head_cursor[slot] = pos;
      if (j % n_classes == 0 && slot / n_classes == qx) sched[qx] = pos;  // first head of queue qx
      pos += s_hist[slot];
    }
    __syncthreads();  // every queue's first position is in sched
    if (tid == 0) {
      int32_t total = 0;
      for (int w = 0; w < kScanThreads / 64; ++w) total += s_rows[w];
      // queues without heads (fewer than 8 heads) are empty and sit at the end
      for (int x = num_heads; x < kXcds; ++x) sched[x] = total;
      sched[kXcds] = total;
      for (int i = kXcds + 1; i < 32; ++i) sched[i] = 0;
      sched[25] = max_n;
      // A queue's rows go to the cus_per_xcd workgroups of its XCD.  When there are so few rows that
      // at most half of the workgroups would get one, every row is cut into 2..4 parts (consecutive
      // ranges of its kv blocks) so that they all get work.  (With one or more full rounds of rows
      // the parts' extra prologues and the merge cost what the better balance gains: measured.)
      int32_t slot = 0;
      for (int x = 0; x < kXcds; ++x) {
        const int32_t len = sched[x + 1] - sched[x];
        int32_t rest = 0, parts = 1;
        if (cus_per_xcd > 1) {
          const int32_t rounds = len / cus_per_xcd, rem = len - rounds * cus_per_xcd;
          if (rounds < kSplitMaxRounds && rem > 0 && 2 * rem <= cus_per_xcd &&
              slot + rem <= kMaxSplitSlots) {
            rest = rem;
            parts = min(kMaxSplitParts, cus_per_xcd / rem);
          }
        }
        sched[kSchedSplitStart + x] = sched[x + 1] - rest;
        sched[kSchedSplitParts + x] = parts;
        sched[kSchedSplitSlot + x] = slot;
        slot += rest;
      }
    }
    for (int i = tid; i < kMaxSplitSlots; i += kScanThreads) sched[kSchedArrived + i] = 0;
  }
}

__global__ void __launch_bounds__(kCountThreads) decode_fill_kernel(
    const uint8_t* __restrict__ sparse_info, const uint8_t* __restrict__ sparse_kv_info,
    const int32_t* __restrict__ sparse_info_indptr,
    const int32_t* __restrict__ sparse_kv_info_indptr, const int32_t* __restrict__ blk_req,
    const int32_t* __restrict__ blk_qb, const int32_t* __restrict__ kv_indptr, int64_t n_cand,
    int32_t num_heads, int32_t block_kv, int is_full, const int32_t* __restrict__ row_pos,
    const int32_t* __restrict__ kv_pos, int32_t* __restrict__ row_req,
    int32_t* __restrict__ row_qb, int32_t* __restrict__ row_head,
    int32_t* __restrict__ kv_row_ptr, int32_t* __restrict__ kv_idx,
    int32_t* __restrict__ head_cursor, int32_t* __restrict__ order,
    const int32_t* __restrict__ counts, const int32_t* __restrict__ sched) {
  const int lane = threadIdx.x % kWave;
  const int64_t c = static_cast<int64_t>(blockIdx.x) * (kCountThreads / kWave) + threadIdx.x / kWave;
  if (c >= n_cand) return;
  const int32_t pos = row_pos[c];
  if (pos < 0) return;
  const Candidate cd = load_candidate(c, num_heads, block_kv, is_full, sparse_info,
                                      sparse_info_indptr, blk_req, blk_qb, kv_indptr);
  int32_t out = kv_pos[c];
  if (lane == 0) {
    row_req[pos] = cd.req;
    row_qb[pos] = cd.qb;
    row_head[pos] = cd.head;
    kv_row_ptr[pos] = out;
    const int32_t listed = (c + 1 < n_cand ? kv_pos[c + 1] : counts[1]) - out;  // kv blocks of this row
    const int n_classes = len_classes(num_heads);
    order[atomicAdd(&head_cursor[cd.head * n_classes + len_class(listed, sched[25], n_classes)], 1)] = pos;
  }
  if (cd.nkv <= 0) return;
  if (is_full) {
    for (int32_t j = lane; j < cd.nkv; j += kWave) kv_idx[out + j] = j;
    return;
  }
  const uint8_t* seg = sparse_kv_info + sparse_kv_info_indptr[cd.req];
  const int64_t b0 = cd.base >> 3, b1 = (cd.base + cd.nkv - 1) >> 3;
  for (int64_t bb = b0; bb <= b1; bb += kWave) {  // uniform trip count for the whole wave
    const int64_t b = bb + lane;
    uint32_t m = (b <= b1) ? masked_byte(seg, b, cd.base, cd.nkv) : 0u;
    const int32_t pc = __popc(m);
    int32_t incl = pc;
    for (int off = 1; off < kWave; off <<= 1) {
      const int32_t up = __shfl_up(incl, off, kWave);
      if (lane >= off) incl += up;
    }
    int32_t w = out + incl - pc;
    while (m) {
      const int p = __ffs(m) - 1;
      m &= m - 1;
      kv_idx[w++] = static_cast<int32_t>(b * 8 + p - cd.base);
    }
    out += __shfl(incl, kWave - 1, kWave);
  }
}

}  // namespace

extern "C" int fo_decode_sparse(const uint8_t* sparse_info, const uint8_t* sparse_kv_info,
                                const int32_t* sparse_info_indptr,
                                const int32_t* sparse_kv_info_indptr, const int32_t* blk_req,
                                const int32_t* blk_qb, const int32_t* kv_indptr, int32_t n_blk,
                                int32_t num_heads, int32_t block_kv, int is_full,
                                int32_t* row_req, int32_t* row_qb, int32_t* row_head,
                                int32_t* kv_row_ptr, int32_t* kv_idx, int32_t* counts,
                                int32_t* order, int32_t* sched, int32_t* scratch, int split_rows,
                                void* stream) {
  FO_REQUIRE(n_blk >= 0 && num_heads > 0 && num_heads <= kMaxHeads && block_kv > 0,
             "decode: bad sizes");
  FO_REQUIRE(counts && kv_row_ptr && order && sched, "decode: null output");
  if (!is_full) {
    FO_REQUIRE(sparse_info && sparse_kv_info && sparse_info_indptr && sparse_kv_info_indptr,
               "decode: sparse_info, sparse_kv_info and their indptrs are required unless is_full");
  }
  FO_REQUIRE(blk_req && blk_qb && kv_indptr && scratch, "decode: null table");
  const int64_t n_cand = static_cast<int64_t>(n_blk) * num_heads;
  FO_REQUIRE(n_cand < (int64_t(1) << 31), "decode: too many (q-block, head) pairs");
  hipStream_t s = static_cast<hipStream_t>(stream);
  int32_t* act = scratch;
  int32_t* cnt = scratch + n_cand;
  int32_t* head_cursor = scratch + 2 * n_cand;
  if (n_cand > 0) {
    FO_REQUIRE(row_req && row_qb && row_head && kv_idx, "decode: null output");
    const int per_wg = kCountThreads / kWave;
    const unsigned grid = static_cast<unsigned>((n_cand + per_wg - 1) / per_wg);
    decode_count_kernel<<<grid, kCountThreads, 0, s>>>(
        sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr, blk_req, blk_qb,
        kv_indptr, n_cand, num_heads, block_kv, is_full, act, cnt);
    FO_CHECK_LAUNCH();
  }
  const int32_t cus_per_xcd = split_rows ? fo_num_cu() / kXcds : 0;
  decode_scan_kernel<<<1, kScanThreads, 0, s>>>(n_cand, num_heads, act, cnt, kv_row_ptr, counts,
                                                head_cursor, sched, cus_per_xcd);
  FO_CHECK_LAUNCH();
  if (n_cand > 0) {
    const int per_wg = kCountThreads / kWave;
    const unsigned grid = static_cast<unsigned>((n_cand + per_wg - 1) / per_wg);
    decode_fill_kernel<<<grid, kCountThreads, 0, s>>>(
        sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr, blk_req, blk_qb,
        kv_indptr, n_cand, num_heads, block_kv, is_full, act, cnt, row_req, row_qb, row_head,
        kv_row_ptr, kv_idx, head_cursor, order, counts, sched);
    FO_CHECK_LAUNCH();
  }
  return FO_OK;
}
