// Sparse-symbol decoder for gfx950: bit-packed (head, q-block) flags and (head, q-block, kv-block)
// keep masks -> compacted work list in canonical order (ascending request, q-block, head; kv
// blocks ascending inside a row).  Lists of up to 1024 (q-block, head) candidates are decoded by one
// launch of one workgroup (decode_small_kernel); longer ones by three short launches on one stream,
// no host round trip:
//   count : one wavefront per (q-block, head) candidate; lanes take one mask byte each, popcount
//   scan  : one workgroup, exclusive prefix sums of row flags and kv counts (canonical positions),
//           plus a per-head histogram that lays out the execution order
//   fill  : one wavefront per candidate again; wave prefix of popcounts places every kv index
//
// Besides the canonical list the decoder emits an execution order for the attention kernel:
// `order` lists row positions grouped by head, heads dealt to the 8 XCDs round-robin (head % 8), so
// that the workgroups of one XCD (which share an L2) walk the rows of the same few heads and find
// that head's K/V in their L2.  Inside a head the order depends on how long the list is:
//   * eight or more rows per workgroup of the attention kernel: q blocks ascending (a fixed order,
//     laid out by the scan kernel).  Neighbouring q blocks of a head keep overlapping kv blocks
//     (windowed masks), so the workgroups of an XCD, which pop consecutive entries, share K/V tiles
//     in that XCD's L2; with that many rows per workgroup the finishing times even out by themselves;
//   * fewer: longest rows first (up to 32 length classes relative to the longest row of the launch),
//     which evens out the workgroups' finishing times; the order inside a length class is not
//     deterministic (atomic cursors), results do not depend on it;
//   * at most two rows per workgroup (and a share table to fill): "even shares", see the scan kernel.
// sched[0..8] delimit the 8 per-XCD queues inside `order`, sched[16..23] are the queue cursors,
// sched[24] a completion counter (all cleared here) and sched[25] the longest row's kv count.
// Integer work, bounded by HBM traffic and launch latency; bit-exact by construction.
//
// Symbol semantics (reference: include/flashomni/attention/prefill.cuh:1284-1294, 1380-1403,
// 1434-1460): bit 1 = compute/keep, little-endian bytes, flag bit index qb*H + h, keep-mask bit
// index (qb*H + h)*NKV + kvb, per-request byte offsets.
#include <mutex>

#include "fo_common.h"

namespace {

constexpr int kWave = 64;
constexpr int kCountThreads = 256;  // 4 candidates per workgroup
constexpr int kScanThreads = 1024;
constexpr int kMaxHeads = 1024;
constexpr int kXcds = 8;
constexpr int kHistSlots = 8192;  // (head, length class) counters of the order layout
// even shares (see the attention kernel): words of `sched` and limits
constexpr int kSchedEven = 26, kSchedShare = 27, kSchedTotal = 28, kSchedShares = 29, kSchedRows = 30,
              kSchedRecords = 31, kSchedOrdered = 32, kSchedArrived = 64;
constexpr int kSchedWords = 40;      // words [0, kSchedWords) are rewritten by every decode
constexpr int kRecordInts = 8;  // queue entry: row, request, q block, head, first kv slot, kv count, pad, pad
constexpr int kMaxShares = 512;      // arrival counters in `sched`, first-row entries in `shares`
constexpr int kMaxSplitParts = 4;    // a row is cut into at most this many parts
constexpr int kEvenMaxRounds = 2;    // even shares when there are at most this many rows per workgroup.
// (Measured: at 2.5 rows per workgroup even shares are 2 % ahead of the queues but miss the L2 3.7 times as
// often, three heads' K and V being live in every XCD at once; from ~5 rows on the queues balance as well and
// adapt to the workgroups' actual speeds, which fixed shares cannot.)
constexpr int kRowOverhead = 3;      // fixed cost of a row (prologue, epilogue) in units of one kv block
constexpr int kOrderedMinRounds = 8; // q blocks ascending inside a head from this many rows per workgroup on

// number of length classes for num_heads heads (32 up to 256 heads)
__host__ __device__ __forceinline__ int len_classes(int32_t num_heads) {
  const int k = kHistSlots / num_heads;
  return k > 32 ? 32 : k;
}
// length class of a row with n kv blocks when the longest row has max_n: 0 = longest
__device__ __forceinline__ int len_class(int32_t n, int32_t max_n, int n_classes) {
  // (n_classes <= 32: the product fits 32 bits below 2^26 blocks, and a 64-bit division costs an order
  // of magnitude more instructions than a 32-bit one)
  if (max_n < (1 << 26)) return static_cast<int>(static_cast<uint32_t>(max_n - n) * n_classes / static_cast<uint32_t>(max_n + 1));
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
  const int32_t t = static_cast<int32_t>(c) / num_heads;  // (fewer than 2^31 candidates)
  cd.head = static_cast<int32_t>(c) - t * num_heads;
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

// Inclusive prefix sum over the 64 lanes of a wavefront.  Rows of 16 lanes by data-parallel lane
// shifts (vector ALU speed; lanes shifted in from outside a row read zero), then the three row
// totals through scalar registers.  (Lane shuffles go through the LDS unit, which the sixteen
// wavefronts of a scan workgroup share: 12 per value made that unit the scan's bottleneck.)
__device__ __forceinline__ int32_t wave_scan(int32_t v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);  // row_shr:8
  const int32_t t0 = __builtin_amdgcn_readlane(v, 15), t1 = __builtin_amdgcn_readlane(v, 31),
                t2 = __builtin_amdgcn_readlane(v, 47);
  const int row = (threadIdx.x & 63) >> 4;
  return v + (row >= 1 ? t0 : 0) + (row >= 2 ? t1 : 0) + (row >= 3 ? t2 : 0);
}

// Inclusive prefix sums of (r, k) over the threads of a workgroup of kScanThreads, in thread order:
// wavefront scans by lane shifts, then the sixteen wavefront totals through tot[0..31].  Every
// thread of the workgroup calls it.
__device__ __forceinline__ void workgroup_scan2(int32_t& r, int32_t& k, int32_t* tot) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  r = wave_scan(r);
  k = wave_scan(k);
  if (lane == 63) {
    tot[wave] = r;
    tot[16 + wave] = k;
  }
  __syncthreads();
  for (int w = 0; w < wave; ++w) {
    r += tot[w];
    k += tot[16 + w];
  }
  __syncthreads();
}

// In place: act[c] -> canonical row position (or -1), cnt[c] -> first kv_idx slot of the row.
// One workgroup of kScanThreads threads; every thread returns from the same place.
__device__ __forceinline__ void scan_body(
    int64_t n_cand, int32_t num_heads, int32_t* act, int32_t* cnt, int32_t* kv_row_ptr, int32_t* counts,
    int32_t* head_cursor, int32_t* sched, int32_t* order, int32_t* shares, int32_t n_shares, int32_t n_wg,
    int32_t* s_rows, int32_t* s_kv, int32_t* s_hist, int32_t* s_max_ptr) {
  // s_rows, s_kv [kScanThreads], s_hist [kHistSlots], s_max_ptr [1]: LDS of the calling kernel;
  // head_cursor may be s_hist itself (every slot is read before its own cursor is written)
  int32_t& s_max = *s_max_ptr;
  const int tid = threadIdx.x;
  const int n_classes = len_classes(num_heads);
  for (int h = tid; h < num_heads * n_classes; h += kScanThreads) s_hist[h] = 0;
  if (tid == 0) s_max = 0;
  __syncthreads();
  // Every pass walks the candidates in tiles of 1024, thread i taking candidate tile + i: neighbouring
  // lanes read neighbouring words (a thread-per-chunk walk costs a cache line per lane and load).  One
  // workgroup is latency bound, so a pass takes kBatch tiles at a time: their loads are in flight
  // together and the barriers are shared.
  constexpr int kBatch = 8;
  const int lane = tid & 63, wave = tid >> 6;
  const int32_t n_c = static_cast<int32_t>(n_cand);
  int32_t mx = 0;
  for (int32_t base = 0; base < n_c; base += kBatch * kScanThreads) {
    int32_t v[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int32_t c = base + u * kScanThreads + tid;
      v[u] = c < n_c ? cnt[c] : 0;
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) mx = max(mx, v[u]);
  }
  for (int off = 32; off > 0; off >>= 1) mx = max(mx, __shfl_xor(mx, off, 64));
  if (lane == 0) atomicMax(&s_max, mx);
  __syncthreads();
  const int32_t max_n = s_max;
  // histogram of (head, length class) and the exclusive prefix sums of flags and counts: wavefront
  // scans by lane shifts, the batch's 8 x 16 wavefront totals scanned by the first wavefront, a
  // running carry
  int32_t carry_rows = 0, carry_kv = 0;
  for (int32_t base = 0; base < n_c; base += kBatch * kScanThreads) {
    int32_t a[kBatch], n[kBatch], ia[kBatch], in[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int32_t c = base + u * kScanThreads + tid;
      a[u] = c < n_c ? act[c] : 0;
      n[u] = c < n_c ? cnt[c] : 0;
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int32_t c = base + u * kScanThreads + tid;
      ia[u] = 0;
      in[u] = 0;
      if (base + u * kScanThreads < n_c) {  // (uniform: tiles behind the last candidate are skipped)
        if (a[u]) atomicAdd(&s_hist[(c % num_heads) * n_classes + len_class(n[u], max_n, n_classes)], 1);
        ia[u] = wave_scan(a[u]);
        in[u] = wave_scan(n[u]);
      }
      if (lane == 63) {
        s_rows[u * 16 + wave] = ia[u];
        s_kv[u * 16 + wave] = in[u];
      }
    }
    __syncthreads();
    if (wave == 0) {  // the 128 totals, two per lane -> their exclusive prefix sums (carry included)
      const int32_t r0 = s_rows[2 * lane], r1 = s_rows[2 * lane + 1];
      const int32_t k0 = s_kv[2 * lane], k1 = s_kv[2 * lane + 1];
      const int32_t ir = wave_scan(r0 + r1), ik = wave_scan(k0 + k1);
      const int32_t er = carry_rows + ir - (r0 + r1), ek = carry_kv + ik - (k0 + k1);
      s_rows[2 * lane] = er;
      s_rows[2 * lane + 1] = er + r0;
      s_kv[2 * lane] = ek;
      s_kv[2 * lane + 1] = ek + k0;
      if (lane == 63) {
        s_rows[kBatch * 16] = carry_rows + ir;
        s_kv[kBatch * 16] = carry_kv + ik;
      }
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int32_t c = base + u * kScanThreads + tid;
      if (c < n_c) {
        act[c] = a[u] ? s_rows[u * 16 + wave] + ia[u] - a[u] : -1;
        cnt[c] = s_kv[u * 16 + wave] + in[u] - n[u];
      }
    }
    carry_rows = s_rows[kBatch * 16];
    carry_kv = s_kv[kBatch * 16];
    __syncthreads();  // (the totals are read before the next batch writes its own)
  }
  const int32_t n_rows = carry_rows, nnz = carry_kv;
  if (tid == kScanThreads - 1) {
    counts[0] = n_rows;
    counts[1] = nnz;
    counts[2] = 0;
    counts[3] = 0;
    kv_row_ptr[n_rows] = nnz;
  }
  __threadfence_block();
  __syncthreads();  // s_rows / s_kv are free again; act / cnt hold positions now

  // Even shares.  With only a few rows per workgroup, whole rows cannot be dealt evenly (at 2.5 rows
  // per workgroup the last one to finish has three while others have two).  The rows are then laid
  // out head by head (q blocks ascending inside a head: a fixed order), every row costs
  // kRowOverhead + its kv blocks, and workgroup j of the attention kernel gets the cost range
  // [j * share, (j + 1) * share): rows that straddle a boundary are computed in parts by the
  // neighbouring workgroups and combined by whoever finishes last.  Nothing depends on timing, so
  // results repeat from launch to launch.
  const bool even = shares != nullptr && n_shares > 0 && n_shares <= kMaxShares && n_rows > 0 &&
                    n_rows <= kEvenMaxRounds * n_shares && num_heads <= kScanThreads;
  if (even) {
    const int32_t nq = static_cast<int32_t>(n_cand / num_heads);
    const int segs = kScanThreads / num_heads;  // threads per head, each a run of q blocks
    const int per = (nq + segs - 1) / segs;
    // (neighbouring threads take neighbouring heads of one run: neighbouring words of act / cnt)
    const int seg = tid / num_heads, h = tid - seg * num_heads;
    const bool mine = seg < segs;
    const int slot = mine ? h * segs + seg : 0;  // layout order: head by head, a head's runs in order
    const int t0 = mine ? min(seg * per, nq) : 0, t1 = mine ? min(t0 + per, nq) : 0;
    auto kv_count = [&](int64_t c) { return (c + 1 < n_cand ? cnt[c + 1] : nnz) - cnt[c]; };
    int32_t my_rows = 0, my_cost = 0;
    for (int t = t0; t < t1; ++t) {
      const int64_t c = static_cast<int64_t>(t) * num_heads + h;
      if (act[c] >= 0) {
        ++my_rows;
        my_cost += kRowOverhead + kv_count(c);
      }
    }
    s_rows[tid] = 0;
    s_kv[tid] = 0;
    __syncthreads();
    if (mine) {  // (the slots of the runs are a permutation of the first H * segs)
      s_rows[slot] = my_rows;
      s_kv[slot] = my_cost;
    }
    __syncthreads();
    {
      int32_t r = s_rows[tid], k = s_kv[tid];
      workgroup_scan2(r, k, s_hist);  // (the histogram is not used on this path)
      s_rows[tid] = r;
      s_kv[tid] = k;
      __syncthreads();
    }
    const int32_t total = s_kv[kScanThreads - 1];
    // a row of n blocks touches at most ceil(n / share) + 1 ranges: share >= n / 3 keeps that within
    // kMaxSplitParts
    static_assert(kMaxSplitParts == 4, "the share's lower bound assumes four parts");
    const int32_t share = max(max((total + n_shares - 1) / n_shares, (max_n + 2) / 3), 1);
    int32_t pos = s_rows[slot] - my_rows, cost = s_kv[slot] - my_cost;
    int32_t* first_row = shares;           // [kMaxShares]
    int32_t* row_start = shares + kMaxShares;  // [n_rows + 1]: cost at which a row's kv blocks begin
    for (int t = t0; t < t1; ++t) {
      const int64_t c = static_cast<int64_t>(t) * num_heads + h;
      if (act[c] >= 0) {
        order[pos] = act[c];
        row_start[pos] = cost + kRowOverhead;
        // first row of a share: the first one whose cost ends behind the share's lower bound
        // j * share, i.e. the row whose cost range [cost, after) holds it (a row without kv blocks
        // stands for the last unit of its own overhead)
        const int32_t after = cost + kRowOverhead + kv_count(c);
        for (int32_t j = (cost + share - 1) / share; j < n_shares && j * share < after; ++j) first_row[j] = pos;
        ++pos;
        cost = after;
      }
    }
    // (shares that begin behind the last row)
    for (int32_t j = (total + share - 1) / share + tid; j < n_shares; j += kScanThreads) first_row[j] = n_rows;
    if (tid == 0) {
      row_start[n_rows] = total + kRowOverhead;
      for (int i = 0; i < kSchedWords; ++i) sched[i] = 0;
      // (the queues stay usable: eight equal runs of the same order, for a launch without shares)
      for (int x = 0; x <= kXcds; ++x) sched[x] = static_cast<int32_t>(static_cast<int64_t>(n_rows) * x / kXcds);
      sched[25] = max_n;
      sched[kSchedEven] = 1;
      sched[kSchedShare] = share;
      sched[kSchedTotal] = total;
      sched[kSchedShares] = n_shares;
      sched[kSchedRows] = n_rows;
    }
    for (int i = tid; i < kMaxShares; i += kScanThreads) sched[kSchedArrived + i] = 0;
    return;
  }

  // Long lists: queue x holds heads x, x+8, x+16, ... back to back, every head's rows with q blocks
  // ascending.  Each head is cut into runs of q blocks, one per thread; the runs are numbered in queue
  // order, so one prefix sum over the threads' row counts places every row.
  if (n_wg > 0 && n_rows >= kOrderedMinRounds * n_wg && num_heads <= kScanThreads) {
    const int32_t nq = static_cast<int32_t>(n_cand / num_heads);
    const int segs = kScanThreads / num_heads;
    const int per = (nq + segs - 1) / segs;
    // (neighbouring threads take neighbouring heads of one run: neighbouring words of act / cnt)
    const int seg = tid / num_heads, h = tid - seg * num_heads;
    const bool mine = seg < segs;
    auto heads_of_queue = [&](int x) { return num_heads > x ? (num_heads - x + kXcds - 1) / kXcds : 0; };
    auto queue_base = [&](int x) {  // heads in the queues before queue x
      int b = 0;
      for (int y = 0; y < x; ++y) b += heads_of_queue(y);
      return b;
    };
    const int t0 = mine ? min(seg * per, nq) : 0, t1 = mine ? min(t0 + per, nq) : 0;
    int32_t my_rows = 0;
    for (int t = t0; t < t1; ++t) my_rows += act[static_cast<int64_t>(t) * num_heads + h] >= 0 ? 1 : 0;
    s_rows[tid] = 0;
    __syncthreads();
    const int slot = mine ? (queue_base(h % kXcds) + h / kXcds) * segs + seg : 0;
    if (mine) s_rows[slot] = my_rows;  // (the slots of the heads' runs are a permutation of the first H * segs)
    __syncthreads();
    {
      int32_t r = s_rows[tid], k = 0;
      workgroup_scan2(r, k, s_hist);  // (the histogram is not used on this path)
      s_rows[tid] = r;
      __syncthreads();
    }
    // first queue position of every run, at [run * num_heads + head]: the fill kernel adds a row's rank
    // inside its run (a thread per run writing the run's rows here costs a dependent trip to memory
    // per row of the run)
    if (mine) head_cursor[tid] = s_rows[slot] - my_rows;
    if (tid == 0) {
      for (int i = 0; i < kSchedWords; ++i) sched[i] = 0;
      for (int x = 0; x <= kXcds; ++x) {
        const int first = queue_base(x) * segs;  // first run of queue x (x = 8: one past the last)
        sched[x] = first > 0 ? s_rows[first - 1] : 0;
      }
      sched[25] = max_n;
      sched[kSchedRecords] = shares != nullptr ? 1 : 0;
      sched[kSchedOrdered] = 1;  // the fill kernel places a row by its run and its rank in the run
    }
    return;
  }

  // shorter lists: queue x holds heads x, x+8, x+16, ... back to back, each head's length
  // classes in order.  Exclusive prefix sum of the histogram taken in that order: every thread owns
  // a run of consecutive entries, wavefront scan by lane shifts, then the sixteen wavefront totals.
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
    const int32_t incl = wave_scan(mine);
    if (lane == 63) s_rows[wave] = incl;
    __syncthreads();
    int32_t pos = incl - mine;
    for (int w = 0; w < wave; ++w) pos += s_rows[w];
    for (int j = e_lo; j < e_hi; ++j) {
      const int slot = slot_of(j, &qx);
      const int32_t n_slot = s_hist[slot];
      head_cursor[slot] = pos;
      if (j % n_classes == 0 && slot / n_classes == qx) sched[qx] = pos;  // first head of queue qx
      pos += n_slot;
    }
    __syncthreads();  // every queue's first position is in sched
    if (tid == 0) {
      int32_t total = 0;
      for (int w = 0; w < kScanThreads / 64; ++w) total += s_rows[w];
      // queues without heads (fewer than 8 heads) are empty and sit at the end
      for (int x = num_heads; x < kXcds; ++x) sched[x] = total;
      sched[kXcds] = total;
      for (int i = kXcds + 1; i < kSchedWords; ++i) sched[i] = 0;
      sched[25] = max_n;
      // with a share table the fill kernel also leaves one record per queue entry there (what the
      // attention kernel needs to start a row: one load after the pop instead of three rounds)
      sched[kSchedRecords] = shares != nullptr ? 1 : 0;
    }
  }
}

__global__ void __launch_bounds__(kScanThreads) decode_scan_kernel(
    int64_t n_cand, int32_t num_heads, int32_t* __restrict__ act, int32_t* __restrict__ cnt,
    int32_t* __restrict__ kv_row_ptr, int32_t* __restrict__ counts,
    int32_t* __restrict__ head_cursor, int32_t* __restrict__ sched, int32_t* __restrict__ order,
    int32_t* __restrict__ shares, int32_t n_shares, int32_t n_wg) {
  __shared__ int32_t s_rows[kScanThreads];
  __shared__ int32_t s_kv[kScanThreads];
  __shared__ int32_t s_hist[kHistSlots];
  __shared__ int32_t s_max;
  scan_body(n_cand, num_heads, act, cnt, kv_row_ptr, counts, head_cursor, sched, order, shares, n_shares, n_wg,
            s_rows, s_kv, s_hist, &s_max);
}

// Short lists (at most one candidate per thread of one workgroup): count, scan and fill in one launch,
// a thread per candidate.  Three launches of a few microseconds each cost more in launch gaps than
// in work; here the candidates' loads are all in flight together and the phases are separated by
// workgroup barriers.  Same outputs as the three kernels.
__global__ void __launch_bounds__(kScanThreads) decode_small_kernel(
    const uint8_t* __restrict__ sparse_info, const uint8_t* __restrict__ sparse_kv_info,
    const int32_t* __restrict__ sparse_info_indptr, const int32_t* __restrict__ sparse_kv_info_indptr,
    const int32_t* __restrict__ blk_req, const int32_t* __restrict__ blk_qb,
    const int32_t* __restrict__ kv_indptr, int64_t n_cand, int32_t num_heads, int32_t block_kv, int is_full,
    int32_t* row_req, int32_t* row_qb, int32_t* row_head, int32_t* kv_row_ptr, int32_t* kv_idx,
    int32_t* counts, int32_t* order, int32_t* sched, int32_t* shares, int32_t n_shares, int32_t n_wg) {
  // (flags, counts and cursors stay in LDS: every trip to memory between the phases costs about as
  // much as a phase's arithmetic)
  __shared__ int32_t s_rows[kScanThreads];
  __shared__ int32_t s_kv[kScanThreads];
  __shared__ int32_t s_hist[kHistSlots];
  __shared__ int32_t s_max;
  __shared__ int32_t act[kScanThreads];
  __shared__ int32_t cnt[kScanThreads];
  __shared__ int32_t s_nnz;
  int32_t* const head_cursor = s_hist;
  const int64_t c = threadIdx.x;
  Candidate cd{};
  const uint8_t* seg = nullptr;
  int64_t b0 = 0, b1 = -1;
  uint64_t bits = 0;    // the row's keep bits when they fit eight mask bytes: read once, used twice
  bool packed = false;
  if (c < n_cand) {
    cd = load_candidate(c, num_heads, block_kv, is_full, sparse_info, sparse_info_indptr, blk_req, blk_qb, kv_indptr);
    int32_t total = 0;
    if (cd.active) {
      if (is_full) {
        total = cd.nkv;
      } else if (cd.nkv > 0) {
        seg = sparse_kv_info + sparse_kv_info_indptr[cd.req];
        b0 = cd.base >> 3;
        b1 = (cd.base + cd.nkv - 1) >> 3;
        packed = (cd.base & 7) + cd.nkv <= 64;
        if (packed) {
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (b0 + u <= b1) bits |= static_cast<uint64_t>(seg[b0 + u]) << (8 * u);
          bits >>= cd.base & 7;
          if (cd.nkv < 64) bits &= (uint64_t(1) << cd.nkv) - 1;
          total = __popcll(bits);
        } else {
          for (int64_t b = b0; b <= b1; ++b) total += __popc(masked_byte(seg, b, cd.base, cd.nkv));
        }
      }
    }
    act[c] = cd.active ? 1 : 0;
    cnt[c] = total;
  }
  __syncthreads();
  scan_body(n_cand, num_heads, act, cnt, kv_row_ptr, counts, head_cursor, sched, order, shares, n_shares, n_wg,
            s_rows, s_kv, s_hist, &s_max);
  __syncthreads();
  // (what the fill needs of the scan's results in memory, read once: the writes of other threads
  // of this workgroup are visible after the barrier)
  if (threadIdx.x == 0) s_nnz = counts[1];
  const int32_t max_n = sched[25];
  const bool order_done = sched[kSchedEven] != 0;
  const bool ordered = sched[kSchedOrdered] != 0;
  __syncthreads();
  if (c >= n_cand) return;
  const int32_t pos = act[c];
  if (pos < 0) return;
  const int32_t out = cnt[c];
  row_req[pos] = cd.req;
  row_qb[pos] = cd.qb;
  row_head[pos] = cd.head;
  kv_row_ptr[pos] = out;
  const int32_t listed = (c + 1 < n_cand ? cnt[c + 1] : s_nnz) - out;  // kv blocks of this row
  if (!order_done) {  // (otherwise the scan has written the order)
    const int n_classes = len_classes(num_heads);
    // (rows in runs: with a thread per candidate every run is one q block, so a row is its run's first)
    const int32_t at = ordered ? head_cursor[c]
                               : atomicAdd(&head_cursor[cd.head * n_classes + len_class(listed, max_n, n_classes)], 1);
    order[at] = pos;
    if (shares) {
      typedef __attribute__((ext_vector_type(4))) int i32x4;
      i32x4* rec = reinterpret_cast<i32x4*>(shares + kMaxShares + kRecordInts * static_cast<int64_t>(at));
      rec[0] = i32x4{pos, cd.req, cd.qb, cd.head};
      rec[1] = i32x4{out, listed, 0, 0};
    }
  }
  if (is_full) {
    for (int32_t j = 0; j < cd.nkv; ++j) kv_idx[out + j] = j;
    return;
  }
  int32_t w = out;
  if (packed) {
    while (bits) {
      kv_idx[w++] = __ffsll(static_cast<unsigned long long>(bits)) - 1;
      bits &= bits - 1;
    }
    return;
  }
  for (int64_t b = b0; b <= b1; ++b) {
    uint32_t m = masked_byte(seg, b, cd.base, cd.nkv);
    while (m) {
      const int p = __ffs(m) - 1;
      m &= m - 1;
      kv_idx[w++] = static_cast<int32_t>(b * 8 + p - cd.base);
    }
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
    const int32_t* __restrict__ counts, const int32_t* __restrict__ sched,
    int32_t* __restrict__ shares) {
  const int lane = threadIdx.x % kWave;
  const int64_t c = static_cast<int64_t>(blockIdx.x) * (kCountThreads / kWave) + threadIdx.x / kWave;
  if (c >= n_cand) return;
  const int32_t pos = row_pos[c];
  if (pos < 0) return;
  const Candidate cd = load_candidate(c, num_heads, block_kv, is_full, sparse_info,
                                      sparse_info_indptr, blk_req, blk_qb, kv_indptr);
  int32_t out = kv_pos[c];
  // rows in runs (see the scan): queue position = the run's first position + the active rows of the
  // same head at earlier q blocks of the run, counted by the wavefront's lanes
  const bool ordered = sched[kSchedOrdered] != 0;
  int32_t rank = 0, run_first = 0;
  if (ordered) {
    const int segs = kScanThreads / num_heads;
    const int32_t nq = static_cast<int32_t>(n_cand / num_heads), per = (nq + segs - 1) / segs;
    const int32_t t = static_cast<int32_t>(c) / num_heads, run = t / per;
    run_first = head_cursor[run * num_heads + cd.head];
    for (int32_t tb = run * per; tb < t; tb += kWave) {
      const int32_t tt = tb + lane;
      const bool on = tt < t && row_pos[static_cast<int64_t>(tt) * num_heads + cd.head] >= 0;
      rank += __popcll(__ballot(on));
    }
  }
  if (lane == 0) {
    row_req[pos] = cd.req;
    row_qb[pos] = cd.qb;
    row_head[pos] = cd.head;
    kv_row_ptr[pos] = out;
    const int32_t listed = (c + 1 < n_cand ? kv_pos[c + 1] : counts[1]) - out;  // kv blocks of this row
    const int n_classes = len_classes(num_heads);
    if (!sched[kSchedEven]) {  // (otherwise the scan kernel has written the order)
      const int32_t at = ordered ? run_first + rank
                                 : atomicAdd(&head_cursor[cd.head * n_classes + len_class(listed, sched[25], n_classes)], 1);
      order[at] = pos;
      if (shares) {
        typedef __attribute__((ext_vector_type(4))) int i32x4;
        i32x4* rec = reinterpret_cast<i32x4*>(shares + kMaxShares + kRecordInts * static_cast<int64_t>(at));
        rec[0] = i32x4{pos, cd.req, cd.qb, cd.head};
        rec[1] = i32x4{out, listed, 0, 0};
      }
    }
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
    const int32_t incl = wave_scan(pc);
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

// Scratch of the entry point that takes no scratch argument: the per-candidate flags and counts of
// the count kernel (2 * n_blk * H ints) and the per-(head, length class) cursors (8192 ints).  1 MiB per
// device, held until the process ends.
constexpr int64_t kStaticScratchInts = 262144;
static __device__ __align__(256) int32_t scratch[kStaticScratchInts];

namespace {

int decode_impl(const uint8_t* sparse_info, const uint8_t* sparse_kv_info, const int32_t* sparse_info_indptr,
                const int32_t* sparse_kv_info_indptr, const int32_t* blk_req, const int32_t* blk_qb,
                const int32_t* kv_indptr, int32_t n_blk, int32_t num_heads, int32_t block_kv, int is_full,
                int32_t* row_req, int32_t* row_qb, int32_t* row_head, int32_t* kv_row_ptr, int32_t* kv_idx,
                int32_t* counts, int32_t* order, int32_t* sched, int32_t* scratch_ptr, int32_t* shares,
                void* stream) {
  FO_REQUIRE(n_blk >= 0 && num_heads > 0 && num_heads <= kMaxHeads && block_kv > 0,
             "decode: bad sizes");
  FO_REQUIRE(counts && kv_row_ptr && order && sched, "decode: null output");
  if (!is_full) {
    FO_REQUIRE(sparse_info && sparse_kv_info && sparse_info_indptr && sparse_kv_info_indptr,
               "decode: sparse_info, sparse_kv_info and their indptrs are required unless is_full");
  }
  FO_REQUIRE(blk_req && blk_qb && kv_indptr && scratch_ptr, "decode: null table");
  FO_REQUIRE((reinterpret_cast<uintptr_t>(shares) & 15) == 0, "decode: shares must be 16-byte aligned");
  const int64_t n_cand = static_cast<int64_t>(n_blk) * num_heads;
  FO_REQUIRE(n_cand < (int64_t(1) << 31), "decode: too many (q-block, head) pairs");
  hipStream_t s = static_cast<hipStream_t>(stream);
  int32_t* act = scratch_ptr;
  int32_t* cnt = scratch_ptr + n_cand;
  int32_t* head_cursor = scratch_ptr + 2 * n_cand;
  const int32_t n_wg = fo_num_cu();                // workgroups of the attention kernel: one per CU
  const int32_t n_shares = shares ? n_wg : 0;      // one share per workgroup
  if (n_cand > 0 && n_cand <= kScanThreads) {
    FO_REQUIRE(row_req && row_qb && row_head && kv_idx, "decode: null output");
    decode_small_kernel<<<1, kScanThreads, 0, s>>>(
        sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr, blk_req, blk_qb, kv_indptr,
        n_cand, num_heads, block_kv, is_full, row_req, row_qb, row_head, kv_row_ptr, kv_idx, counts, order,
        sched, shares, n_shares, n_wg);
    FO_CHECK_LAUNCH();
    return FO_OK;
  }
  if (n_cand > 0) {
    FO_REQUIRE(row_req && row_qb && row_head && kv_idx, "decode: null output");
    const int per_wg = kCountThreads / kWave;
    const unsigned grid = static_cast<unsigned>((n_cand + per_wg - 1) / per_wg);
    decode_count_kernel<<<grid, kCountThreads, 0, s>>>(
        sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr, blk_req, blk_qb,
        kv_indptr, n_cand, num_heads, block_kv, is_full, act, cnt);
    FO_CHECK_LAUNCH();
  }
  decode_scan_kernel<<<1, kScanThreads, 0, s>>>(n_cand, num_heads, act, cnt, kv_row_ptr, counts,
                                                head_cursor, sched, order, shares, n_shares, n_wg);
  FO_CHECK_LAUNCH();
  if (n_cand > 0) {
    const int per_wg = kCountThreads / kWave;
    const unsigned grid = static_cast<unsigned>((n_cand + per_wg - 1) / per_wg);
    decode_fill_kernel<<<grid, kCountThreads, 0, s>>>(
        sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr, blk_req, blk_qb,
        kv_indptr, n_cand, num_heads, block_kv, is_full, act, cnt, row_req, row_qb, row_head,
        kv_row_ptr, kv_idx, head_cursor, order, counts, sched, shares);
    FO_CHECK_LAUNCH();
  }
  return FO_OK;
}

// device address of `scratch` on the current device (every device holds its own copy of the array
// at its own address); looked up once per device
int static_scratch(int32_t** out) {
  static std::mutex mu;
  static int32_t* ptrs[64] = {};
  int dev = 0;
  FO_HIP_CALL(hipGetDevice(&dev));
  FO_REQUIRE(dev >= 0 && dev < 64, "decode: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (ptrs[dev] == nullptr) {
    void* p = nullptr;
    FO_HIP_CALL(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    FO_REQUIRE(p != nullptr, "decode: the static scratch array has no device address");
    ptrs[dev] = static_cast<int32_t*>(p);
  }
  *out = ptrs[dev];
  return FO_OK;
}

}  // namespace

extern "C" int fo_decode_sparse(const uint8_t* sparse_info, const uint8_t* sparse_kv_info,
                                const int32_t* sparse_info_indptr,
                                const int32_t* sparse_kv_info_indptr, const int32_t* blk_req,
                                const int32_t* blk_qb, const int32_t* kv_indptr, int32_t n_blk,
                                int32_t num_heads, int32_t block_kv, int is_full,
                                int32_t* row_req, int32_t* row_qb, int32_t* row_head,
                                int32_t* kv_row_ptr, int32_t* kv_idx, int32_t* counts,
                                int32_t* order, int32_t* sched, int32_t* scratch, int32_t* shares,
                                void* stream) {
  return decode_impl(sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr, blk_req, blk_qb,
                     kv_indptr, n_blk, num_heads, block_kv, is_full, row_req, row_qb, row_head, kv_row_ptr,
                     kv_idx, counts, order, sched, scratch, shares, stream);
}

extern "C" int64_t fo_decode_sparse_static_max_pairs(void) { return (kStaticScratchInts - kHistSlots) / 2; }

extern "C" int fo_decode_sparse_static(const uint8_t* sparse_info, const uint8_t* sparse_kv_info,
                                       const int32_t* sparse_info_indptr,
                                       const int32_t* sparse_kv_info_indptr, const int32_t* blk_req,
                                       const int32_t* blk_qb, const int32_t* kv_indptr, int32_t n_blk,
                                       int32_t num_heads, int32_t block_kv, int is_full,
                                       int32_t* row_req, int32_t* row_qb, int32_t* row_head,
                                       int32_t* kv_row_ptr, int32_t* kv_idx, int32_t* counts,
                                       int32_t* order, int32_t* sched, int32_t* shares, void* stream) {
  FO_REQUIRE(n_blk >= 0 && num_heads > 0, "decode: bad sizes");
  const int64_t n_cand = static_cast<int64_t>(n_blk) * num_heads;
  FO_REQUIRE(n_cand <= fo_decode_sparse_static_max_pairs(),
             "decode: %lld (q-block, head) pairs exceed the %lld the built-in scratch holds; use "
             "fo_decode_sparse with a caller-provided scratch",
             static_cast<long long>(n_cand), static_cast<long long>(fo_decode_sparse_static_max_pairs()));
  int32_t* ptr = nullptr;
  const int rc = static_scratch(&ptr);
  if (rc != FO_OK) return rc;
  // (nothing in the scratch has to start at zero: the count kernel writes every flag and count the
  // later kernels read, the scan kernel every cursor)
  return decode_impl(sparse_info, sparse_kv_info, sparse_info_indptr, sparse_kv_info_indptr, blk_req, blk_qb,
                     kv_indptr, n_blk, num_heads, block_kv, is_full, row_req, row_qb, row_head, kv_row_ptr,
                     kv_idx, counts, order, sched, ptr, shares, stream);
}
