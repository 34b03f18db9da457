// GEMM-Q and GEMM-O (with reduction) for gfx950: MFMA tile GEMMs that skip work according to the
// bit-packed (token-block, head) flags.
//
//   GEMM-Q  y[b, iy-tile, ix-tile] = x[b, iy-tile, :] . w[ix-tile, :]^T + bias   for flagged tiles;
//           the other tiles are never touched (reference: gemm/w16a16/gemm.cuh:50-58, 83-92).
//   GEMM-O  y[b, iy-tile, :] = init + sum_{selected heads h} x[:, h-slice] . w[:, h-slice]^T
//           where unselected head slices are never loaded
//           (reference: gemm/w16a16/gemm_reduction.cuh:77-95, 126-160).
//
// Tiling.  The skip flags have a 128 x 128 granularity ("unit"), but a CU can pull only ~50-60 B/clk
// from L2 while its matrix cores eat a 128 x 128 x 64 step in ~500 clocks, so small workgroup tiles
// starve.  A workgroup (4 wavefronts, one per SIMD, 512 registers each) therefore computes a *quad*:
// two token blocks x two column blocks that share their operand tiles (four 128 x 64 tiles feed four
// units).  A wavefront owns one unit: 128 x 128 accumulators (256 registers, kept in the accumulator
// half of the register file), sixteen MFMAs per eight 128-bit operand reads.  (With eight wavefronts
// of 64 x 128 the same loop spent a third more LDS reads per MFMA and ran 25 % slower.)  A list
// kernel packs the flagged units of every (16-token-block window, column pair) cell into work items:
// rows flagged in both columns pair up into full quads; rows flagged in one column go three at a time
// into *column strips* (three token blocks x that column block: three X tiles and one W tile, three
// wavefronts busy), what is left pairs up or is merged; a mask says which units of an item exist
// (the wavefront of a missing unit only moves data).  With four fifths of the units flagged at
// random (the 14B-video configuration) that fills 86 % of the wavefront slots against 81 % with
// quads alone, from the same operand tiles, and the launch is 2 % shorter.  (Measured and dropped:
// items dealt by row pair over the whole width, full quads for the columns both token blocks have and
// strips of one token block x three column blocks for the rest: 91 % of the slots, but a strip's
// three columns lie far apart and few concurrent items share its W tiles, 9.4 GB fetched per launch
// against 6.8 GB, and the launch was 1.3 % shorter.  Either way the time per round of work items
// rises with the fill.)  GEMM-O (and GEMM-Q with is_full) computes every unit: no list
// then, the kernel derives its quads from the shape.  GEMM-O walks the union of the two token
// blocks' selected heads; a token block that does not select a head reads that k step's X operand
// as zeros.
//
// Data path.  Operands are staged in slabs of 64 k: a tile row is then 128 B, one whole memory line.
// A wavefront fetches its sixteen 8-row pieces of a slab with buffer loads (a resource descriptor
// per tile in scalar registers, 32-bit lane offsets, the k offset as the scalar offset: no vector
// address arithmetic; rows past M and unselected heads read as zeros through the descriptor's range
// check) into staging registers one slab ahead, and writes them to LDS (two slab buffers) a slab
// later; loads, LDS writes and operand reads are spread evenly between the MFMAs (per sixteen MFMAs:
// eight reads, four writes, four loads), so the memory path sees an even stream and nothing queues
// behind a burst.  (Direct global -> LDS copies need no registers but can only be issued once a
// buffer is free, i.e. in a burst after the barrier: the issue stalls of that burst, 100-150 clocks
// per copy and wavefront, cost a quarter of the loop.)  One barrier per slab.  Rows are XOR-swizzled
// instead of padded: row r keeps logical 16-byte chunk c at position c ^ ((r >> 1) & 7), applied to
// the LDS write address; the 128-bit operand reads of 16 consecutive rows then cover all 64 banks.
// A k range that is not a multiple of 64 (K or the head width of GEMM-O = 32 mod 64) ends in a slab
// that reaches 32 back into its neighbour; that half of its X operand is cleared on the way to LDS
// (a separate instantiation, so that the common case carries no masking).
//
// The product is formed transposed (A operand = W rows, B operand = X rows): in the 32 x 32
// accumulator layout a lane owns one output row and runs of 4 consecutive columns.  Stored (or the
// init matrix read) from that layout, a wavefront instruction is 64 scattered 8-byte pieces, so the
// epilogue turns each wavefront's block through its own quarter of the (by then free) slab buffers,
// 32 rows at a time in fp32, into a layout where 32 consecutive lanes cover one row; there the bias
// vector or the cached partial is added in fp32 and the result is rounded once and stored through a
// buffer descriptor that ends with the matrix (no per-row tests).  The first slab of the next work
// item is requested before the epilogue, so that its latency hides behind the stores (GEMM-O: the
// item's flags are fetched a whole item ahead and its k-step list is built just before that request;
// where a cached partial is added, the request follows the stores, because the partial's pieces need
// the staging registers).
//
// Work order.  Workgroups are persistent (one per CU).  The quad list is ordered by token window,
// then column pair, then row pair, and XCD x (= blockIdx % 8) owns the x-th contiguous eighth of it.
// The ~32 workgroups of an XCD therefore work at the same time on one token window and four
// neighbouring column pairs (16 + 8 operand tiles for 32 quads), whose tiles they share through
// that XCD's L2; work items of equal length keep them in step in k, which is what makes the tiles
// hit (measured at the Wan size: 6.8 GB fetched per launch against 28 GB of operand loads).
#include "fo_common.h"

#include <type_traits>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

constexpr int kThreads = 256;
constexpr int kTile = 128;  // unit edge = granularity of the skip flags
constexpr int kBK = 64;                            // k range of one LDS slab
constexpr int kRowBytes = kBK * 2;                 // one LDS row: 64 elements = one 128-byte memory line, 8 chunks of 16 B
constexpr int kUnitBytes = kTile * kRowBytes;      // one 128-row operand tile: 16 KB
constexpr int kStageBytes = 4 * kUnitBytes;        // X0, X1, W0, W1
constexpr int kStages = 2;
constexpr int kSmemBytes = kStages * kStageBytes;  // 128 KB
constexpr int kZeroFirst = 1 << 18, kZeroSecond = 1 << 19;  // slab entry: half of the slab does not count
constexpr int kMaxHeads = 256;
constexpr int kMaxSteps = 2048;  // GEMM-O: k steps of one work item (K <= 65536)
constexpr int kXcds = 8;
constexpr int kListThreads = 1024;
constexpr int kInlineCells = 256;  // up to this many cells the GEMM-Q kernel lists its quads itself
constexpr int kWindow = 16;   // token blocks per scheduling window
constexpr int kQuadInts = 8;  // b, r0, r1, c0, c1, valid mask, r2 (column strips), pad
constexpr int kColStrip = 0x20;        // in the valid mask: the item is a column strip (three token blocks x one column block)
constexpr int kColStripSecond = 0x40;  // ... of the cell's second column

template <typename T>
struct Types;
template <>
struct Types<__bf16> {
  using x8 = bf16x8;
  using x4 = bf16x4;
  static __device__ __forceinline__ f32x16 mfma(x8 a, x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Types<_Float16> {
  using x8 = f16x8;
  using x4 = f16x4;
  static __device__ __forceinline__ f32x16 mfma(x8 a, x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

struct GemmParams {
  const void* x;     // [B, M, K]
  const void* w;     // [N, K]
  const void* bias;  // [N] or [B, M, N] or null
  void* y;           // [B, M, N]
  const uint8_t* sparse_info;
  const int32_t* sparse_info_indptr;
  const int32_t* quads;  // kQuadInts per quad, queue by queue; null: every unit is computed and the
                         // quads are enumerated arithmetically (GEMM-O, GEMM-Q with is_full)
  const int32_t* qoff;   // qoff[0..8] queue boundaries inside `quads`
  int32_t* cursor;       // GEMM-O, long launches: one work-item cursor per XCD (zero at launch), or null
  int32_t n_row_tiles, n_col_tiles, n_cp;  // geometry for the arithmetic enumeration
  int32_t n_win;         // windows of 16 token blocks per batch
  int32_t inline_cells;  // > 0: GEMM-Q builds its quad list itself from the flags of this many cells
  int32_t batch, m, n, k;
  int32_t sparse_q_size, num_heads, head_dim, num_text_tokens;
  int32_t flag;       // GEMM-Q: is_full.  GEMM-O: is_for_cached
  int32_t bias_kind;  // FO_BIAS_*
  int32_t bias_f32;   // matrix bias is fp32
  int32_t y_f32;      // output is fp32
  // GEMM-Q with fused quantisation: e4m3fn bytes [B, M, N] and one scale per (head, token block),
  // y_scale[head * scale_row_len + b * n_row_tiles + token block]; y may then be null
  uint8_t* y8;
  uint8_t* y8_lo;  // optional second term: the residual result / scale - y8, rounded to e4m3 again
  float* y_scale;
  int32_t scale_row_len;
};

__device__ __forceinline__ bool flag_bit(const uint8_t* info, uint32_t bit) {
  return (info[bit >> 3] >> (bit & 7)) & 1;
}

// ---------------------------------------------------------------------------------------------
// Quad list.  A cell = (batch, window of 16 token blocks, column pair); cells are ordered batch,
// window, column pair.  One workgroup counts the quads of every cell (flagged-row masks of its two
// columns), scans the counts, emits every cell's quads at its offset, and cuts the list into eight
// contiguous, equally long queues.  (Up to kInlineCells cells the GEMM-Q kernel does the same itself.)
// ---------------------------------------------------------------------------------------------
struct ListGeom {
  int32_t batch, n_row_tiles, n_col_tiles, n_win, n_cp;  // windows per batch, column pairs
};

__device__ __forceinline__ void cell_masks(const ListGeom& gm, int cell, bool use_flags,
                                           const uint8_t* __restrict__ sparse_info,
                                           const int32_t* __restrict__ sparse_info_indptr,
                                           int32_t sparse_q_size, int32_t num_heads, int32_t head_dim,
                                           int32_t num_text_tokens, int* b_out, int* row0_out,
                                           int* cp_out, uint32_t* m0, uint32_t* m1) {
  const int cp = cell % gm.n_cp;
  const int t = cell / gm.n_cp;
  const int w = t % gm.n_win, b = t / gm.n_win;
  *b_out = b;
  *row0_out = w * kWindow;
  *cp_out = cp;
  const int rows = min(kWindow, gm.n_row_tiles - w * kWindow);
  const uint32_t all = (1u << rows) - 1u;
  const bool has1 = 2 * cp + 1 < gm.n_col_tiles;
  if (!use_flags) {
    *m0 = all;
    *m1 = has1 ? all : 0u;
    return;
  }
  const uint8_t* info = sparse_info + sparse_info_indptr[b];
  // All flag bytes of the cell are requested before the first is looked at (rows past the end repeat
  // the last one): one memory latency for the cell instead of one per row.
  const uint32_t head0 = static_cast<uint32_t>(2 * cp * kTile) / head_dim;
  const uint32_t head1 = has1 ? static_cast<uint32_t>((2 * cp + 1) * kTile) / head_dim : head0;
  const bool unit_blocks = sparse_q_size == kTile;  // flag blocks = token blocks: no division per row
  const uint32_t text_blocks = static_cast<uint32_t>(num_text_tokens) / kTile;
  uint32_t bit0[kWindow], bit1[kWindow];
  uint8_t byte0[kWindow], byte1[kWindow];
#pragma unroll
  for (int r = 0; r < kWindow; ++r) {
    const int row = w * kWindow + min(r, rows - 1);
    const uint32_t blk = unit_blocks ? text_blocks + static_cast<uint32_t>(row)
                                     : static_cast<uint32_t>(num_text_tokens + row * kTile) / sparse_q_size;
    bit0[r] = blk * num_heads + head0;
    bit1[r] = blk * num_heads + head1;
    byte0[r] = info[bit0[r] >> 3];
    byte1[r] = info[bit1[r] >> 3];
  }
  uint32_t a0 = 0, a1 = 0;
#pragma unroll
  for (int r = 0; r < kWindow; ++r) {
    a0 |= ((byte0[r] >> (bit0[r] & 7)) & 1u) << r;
    a1 |= ((byte1[r] >> (bit1[r] & 7)) & 1u) << r;
  }
  *m0 = a0 & all;
  *m1 = has1 ? a1 & all : 0u;
}

__device__ __forceinline__ int pop_lowest(uint32_t* m) {
  const int r = __ffs(*m) - 1;
  *m &= *m - 1;
  return r;
}

// Packs a cell's flagged units into work items and calls f(r0, r1, valid, r2) for each; r1 < 0 = no
// second row.  Quads: valid bits 1 = (r0,c0), 2 = (r0,c1), 4 = (r1,c0), 8 = (r1,c1).  Column strips
// (col_strips: units come from flags): valid = kColStrip | 7 (| kColStripSecond for the cell's second
// column), rows r0, r1, r2 of that column.
template <typename F>
__device__ __forceinline__ void for_each_quad(uint32_t m0, uint32_t m1, bool col_strips, F&& f) {
  uint32_t both = m0 & m1, only0 = m0 & ~m1, only1 = m1 & ~m0;
  while (__popc(both) >= 2) {
    const int r0 = pop_lowest(&both), r1 = pop_lowest(&both);
    f(r0, r1, 0xF, 0);
  }
  if (col_strips) {
    // rows flagged in one column only: three at a time into a column strip (three X tiles, one W tile)
    while (__popc(only0) >= 3) {
      const int r0 = pop_lowest(&only0), r1 = pop_lowest(&only0), r2 = pop_lowest(&only0);
      f(r0, r1, kColStrip | 0x7, r2);
    }
    while (__popc(only1) >= 3) {
      const int r0 = pop_lowest(&only1), r1 = pop_lowest(&only1), r2 = pop_lowest(&only1);
      f(r0, r1, kColStrip | kColStripSecond | 0x7, r2);
    }
  }
  while (__popc(only0) >= 2) {
    const int r0 = pop_lowest(&only0), r1 = pop_lowest(&only0);
    f(r0, r1, 0x5, 0);
  }
  while (__popc(only1) >= 2) {
    const int r0 = pop_lowest(&only1), r1 = pop_lowest(&only1);
    f(r0, r1, 0xA, 0);
  }
  // at most one row left in each class: merge them two by two
  if (both) {
    const int r0 = pop_lowest(&both);
    if (only0) {
      f(r0, pop_lowest(&only0), 0x3 | 0x4, 0);
    } else if (only1) {
      f(r0, pop_lowest(&only1), 0x3 | 0x8, 0);
    } else {
      f(r0, -1, 0x3, 0);
    }
  }
  if (only0 && only1) {
    const int r0 = pop_lowest(&only0);
    f(r0, pop_lowest(&only1), 0x1 | 0x8, 0);
  } else if (only0) {
    f(pop_lowest(&only0), -1, 0x1, 0);
  } else if (only1) {
    f(pop_lowest(&only1), -1, 0x2, 0);
  }
}

struct ListArgs {
  const uint8_t* sparse_info;
  const int32_t* sparse_info_indptr;
  int32_t use_flags;  // GEMM-Q without is_full: units come from the flags
  int32_t sparse_q_size, num_heads, head_dim, num_text_tokens;
};

__global__ void __launch_bounds__(kListThreads) gemm_quads_kernel(ListArgs a, ListGeom gm,
                                                                  int32_t* __restrict__ quads,
                                                                  int32_t* __restrict__ qoff) {
  __shared__ int32_t s_cnt[kListThreads / 64];
  const int tid = threadIdx.x;
  const int n_cells = gm.batch * gm.n_win * gm.n_cp;
  int b, row0, cp;
  uint32_t m0, m1;
  // every thread owns a contiguous run of cells: quad counts, then a block-wide scan
  const int per = (n_cells + kListThreads - 1) / kListThreads;
  const int lo = min(tid * per, n_cells), hi = min(lo + per, n_cells);
  int32_t my_cnt = 0;
  for (int cell = lo; cell < hi; ++cell) {
    cell_masks(gm, cell, a.use_flags, a.sparse_info, a.sparse_info_indptr, a.sparse_q_size, a.num_heads,
               a.head_dim, a.num_text_tokens, &b, &row0, &cp, &m0, &m1);
    for_each_quad(m0, m1, a.use_flags != 0, [&](int, int, int, int) { ++my_cnt; });
  }
  // inclusive scan of the per-thread counts: inside a wavefront by lane shifts, then over the
  // sixteen wavefront totals
  const int lane = tid & 63, wave = tid >> 6;
  int32_t incl = my_cnt;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int32_t up = __shfl_up(incl, d, 64);
    if (lane >= d) incl += up;
  }
  if (lane == 63) s_cnt[wave] = incl;
  __syncthreads();
  int32_t wave_base = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kListThreads / 64; ++w) {
    const int32_t t = s_cnt[w];
    if (w < wave) wave_base += t;
    total += t;
  }
  const int32_t my_incl = wave_base + incl;
  if (tid <= kXcds) qoff[tid] = static_cast<int32_t>(static_cast<int64_t>(total) * tid / kXcds);
  int32_t q = my_incl - my_cnt;
  for (int cell = lo; cell < hi; ++cell) {
    if (per > 1)  // with one cell per thread the masks of the counting pass are still at hand
      cell_masks(gm, cell, a.use_flags, a.sparse_info, a.sparse_info_indptr, a.sparse_q_size, a.num_heads,
                 a.head_dim, a.num_text_tokens, &b, &row0, &cp, &m0, &m1);
    for_each_quad(m0, m1, a.use_flags != 0, [&](int r0, int r1, int valid, int r2) {
      int32_t* e = quads + kQuadInts * static_cast<int64_t>(q);
      e[0] = b;
      e[1] = row0 + r0;
      e[2] = row0 + (r1 < 0 ? r0 : r1);
      if (valid & kColStrip) {
        e[3] = e[4] = (valid & kColStripSecond) ? 2 * cp + 1 : 2 * cp;
      } else {
        e[3] = (valid & 0x5) ? 2 * cp : 2 * cp + 1;
        e[4] = (valid & 0xA) ? 2 * cp + 1 : 2 * cp;
      }
      e[5] = valid;
      e[6] = row0 + r2;
      ++q;
    });
  }
}

// (the cursors of a launch that hands out its work items dynamically; a kernel, not a memset, so that
// a captured graph replays it faithfully)
__global__ void gemm_cursor_clear_kernel(int32_t* cursor) { cursor[threadIdx.x] = 0; }

// ---------------------------------------------------------------------------------------------
// Main kernel.  kReduce = false: GEMM-Q.  kReduce = true: GEMM-O.  kAux: GEMM-Q with fused
// quantisation / GEMM-O that adds a cached partial (epilogues with register needs of their own).
// ---------------------------------------------------------------------------------------------
template <typename T, bool kReduce, bool kHalf, bool kAux>
__global__ void __launch_bounds__(kThreads) gemm_kernel(const GemmParams p) {
  constexpr bool kQuant = !kReduce && kAux, kPartial = kReduce && kAux;
  using TT = Types<T>;
  using x8 = typename TT::x8;
  using x4 = typename TT::x4;
  constexpr int NT = 4, MT = 4;  // wavefront tile = one unit: 128 columns (W rows) x 128 token rows (X rows)
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  __shared__ int32_t s_popped;
  __shared__ int32_t s_heads[kMaxHeads + 1];  // GEMM-O: head | (row0 selects) << 16 | (row1 selects) << 17
  __shared__ int32_t s_nsel;
  // GEMM-O: per k step, k offset | (row0 selects) << 16 | (row1 selects) << 17; four entries past
  // the end repeat the last step
  __shared__ int32_t s_step[kReduce ? kMaxSteps + 4 : 1];
  // GEMM-Q listing its own quads (short launches: saves the list kernel's launch): quad count
  // prefix and flagged-row masks of every cell, and the entry picked for the current work item
  __shared__ int32_t s_cell_pref[kReduce ? 1 : kInlineCells + 1];
  __shared__ uint32_t s_cell_mask[kReduce ? 1 : 2 * kInlineCells];
  __shared__ int32_t s_cell_wave[kThreads / 64];
  __shared__ int32_t s_entry[8];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);  // wavefront index = unit of the quad, kept scalar
  const int l32 = lane & 31, g = lane >> 5;
  const int wr = wv >> 1, wc = wv & 1;  // token block, column block

  const T* __restrict__ xg = static_cast<const T*>(p.x);
  const T* __restrict__ wg = static_cast<const T*>(p.w);

  // Load assignment: a slab is 64 pieces of 8 rows x 128 B (whole memory lines), 16 per wavefront:
  // pieces 0..7 = rows 64*(wv%2) + 8*j.. of X tile wv/2, pieces 8..15 = the same rows of W tile wv/2.
  // Lane i fetches 16-byte chunk i%8 of row i/8 of its piece and writes it to LDS at chunk position
  // (i%8) ^ ((row >> 1) & 7) = (i%8) ^ ((4*(j%2) + (i >> 4)) & 7).
  const int ld_row = 64 * (wv & 1) + (lane >> 3), ld_chunk = lane & 7;
  int wr_off[2];
#pragma unroll
  for (int par = 0; par < 2; ++par)
    wr_off[par] = (lane >> 3) * kRowBytes + ((ld_chunk ^ ((4 * par + (lane >> 4)) & 7)) << 4);
  // lanes that hold the first / the second half of a slab's k range
  const unsigned mask_first = ld_chunk < 4 ? 0xFFFFFFFFu : 0u;
  // operand reads: row = tile row base + l32 (bases are multiples of 32), logical chunk 2*s + g of substep s
  const int rd_x = (g ^ ((l32 >> 1) & 7)) << 4;

  const int xcd = blockIdx.x & (kXcds - 1), slot = blockIdx.x >> 3;
  const int per_xcd = gridDim.x >> 3;  // host launches a multiple of 8 workgroups
  // dense enumeration (same order as the list kernel's): per batch, windows of 16 token blocks
  // (8 row pairs; the last window may be shorter), column pairs inside a window, row pairs inside
  // a column pair
  const int full_w = p.n_row_tiles / kWindow, last_rows = p.n_row_tiles % kWindow;
  constexpr int per_win = kWindow / 2;  // work items per window and column pair
  const int last_q = (last_rows + 1) / 2;
  const int quads_per_batch = (full_w * per_win + last_q) * p.n_cp;
  int q_lo, q_len;
  bool inline_list = false;
  if constexpr (!kReduce) inline_list = p.inline_cells > 0;
  if (inline_list) {
    if constexpr (!kReduce) {
      // thread = cell: masks, quad count, workgroup-wide inclusive scan of the counts
      ListGeom gm;
      gm.batch = p.batch;
      gm.n_row_tiles = p.n_row_tiles;
      gm.n_col_tiles = p.n_col_tiles;
      gm.n_win = p.n_win;
      gm.n_cp = p.n_cp;
      int32_t cnt = 0;
      if (tid < p.inline_cells) {
        int b, row0, cp;
        uint32_t m0, m1;
        cell_masks(gm, tid, true, p.sparse_info, p.sparse_info_indptr, p.sparse_q_size, p.num_heads,
                   p.head_dim, p.num_text_tokens, &b, &row0, &cp, &m0, &m1);
        for_each_quad(m0, m1, true, [&](int, int, int, int) { ++cnt; });
        s_cell_mask[2 * tid] = m0;
        s_cell_mask[2 * tid + 1] = m1;
      }
      int32_t incl = cnt;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int32_t up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
      }
      if (lane == 63) s_cell_wave[wv] = incl;
      __syncthreads();
      int32_t base = 0, total = 0;
#pragma unroll
      for (int w = 0; w < kThreads / 64; ++w) {
        const int32_t t = s_cell_wave[w];
        if (w < wv) base += t;
        total += t;
      }
      if (tid < kInlineCells) s_cell_pref[tid + 1] = base + incl;
      if (tid == 0) s_cell_pref[0] = 0;
      q_lo = static_cast<int>(static_cast<int64_t>(total) * xcd / kXcds);
      q_len = static_cast<int>(static_cast<int64_t>(total) * (xcd + 1) / kXcds) - q_lo;
      __syncthreads();
    }
  } else if (p.quads) {
    q_lo = p.qoff[xcd];
    q_len = p.qoff[xcd + 1] - q_lo;
  } else {
    const int64_t total = static_cast<int64_t>(quads_per_batch) * p.batch;
    q_lo = static_cast<int>(total * xcd / kXcds);
    q_len = static_cast<int>(total * (xcd + 1) / kXcds) - q_lo;
  }

  // ---- work items ----
  // A work item = a quad: four operand tiles per slab (X r0, X r1, W c0, W c1), wavefront = unit,
  // 128 x 128 each; or a column strip (X r0, X r1, W c0, X r2).  (Another shape was measured and dropped: quads with two units that share a
  // tile, computed by two wavefronts per unit at 64 x 128 each from three tiles.  Its slab takes as
  // long as a full one (nine LDS transfers per eight MFMAs saturate a wavefront's LDS path), and work
  // items of unequal length let the workgroups of an XCD drift apart in k, which costs the L2 hits on
  // the tiles they share.)
  constexpr int P = 16;      // pieces per wavefront and slab: rows 32*wv + 8*jj.. (jj = 0..3) of every tile
  constexpr int PS = P / 4;  // pieces per substep
  // valid & kColStrip (GEMM-Q with flags): the item is a column strip, three token blocks r[0], r[1],
  // r2 x one column block c[0] (tiles: X r[0], X r[1], W c[0], X r2; wavefronts 0..2 own the units).
  struct Item {
    int bz, valid, r[2], c[2], r2;
  };
  // (called by all threads together: the listing form hands the entry over through LDS)
  auto decode_item = [&](int work) -> Item {
    int bz, valid, r[2], c[2], r2 = 0;
    if (inline_list) {
      if constexpr (!kReduce) {
        // the thread whose cell holds quad q_lo + work walks the cell's quads up to it
        const int q = q_lo + work;
        if (tid < p.inline_cells && s_cell_pref[tid] <= q && q < s_cell_pref[tid + 1]) {
          const int cp = tid % p.n_cp, t = tid / p.n_cp;
          const int w = t % p.n_win, b = t / p.n_win;
          int k = q - s_cell_pref[tid];
          for_each_quad(s_cell_mask[2 * tid], s_cell_mask[2 * tid + 1], true, [&](int r0, int r1, int v, int r2) {
            if (k == 0) {
              s_entry[0] = b;
              s_entry[1] = w * kWindow + r0;
              s_entry[2] = w * kWindow + (r1 < 0 ? r0 : r1);
              if (v & kColStrip) {
                s_entry[3] = s_entry[4] = (v & kColStripSecond) ? 2 * cp + 1 : 2 * cp;
              } else {
                s_entry[3] = (v & 0x5) ? 2 * cp : 2 * cp + 1;
                s_entry[4] = (v & 0xA) ? 2 * cp + 1 : 2 * cp;
              }
              s_entry[5] = v;
              s_entry[6] = w * kWindow + r2;
            }
            --k;
          });
        }
        __syncthreads();
        bz = s_entry[0];
        r[0] = s_entry[1];
        r[1] = s_entry[2];
        c[0] = s_entry[3];
        c[1] = s_entry[4];
        valid = s_entry[5];
        r2 = s_entry[6];
      }
    } else if (p.quads) {
      const int32_t* e = p.quads + kQuadInts * static_cast<int64_t>(q_lo + work);
      bz = e[0];
      r[0] = e[1];
      r[1] = e[2];
      c[0] = e[3];
      c[1] = e[4];
      valid = e[5];
      r2 = e[6];
    } else {
      const int q = q_lo + work;
      bz = q / quads_per_batch;
      int rem = q - bz * quads_per_batch;
      int w, cp, i, rows;
      if (rem < full_w * p.n_cp * per_win) {
        const int cell = rem / per_win;
        i = rem - cell * per_win;
        w = cell / p.n_cp;
        cp = cell - w * p.n_cp;
        rows = kWindow;
      } else {
        rem -= full_w * p.n_cp * per_win;
        cp = rem / last_q;
        i = rem - cp * last_q;
        w = full_w;
        rows = last_rows;
      }
      const bool has_r1 = 2 * i + 1 < rows, has_c1 = 2 * cp + 1 < p.n_col_tiles;
      r[0] = w * kWindow + 2 * i;
      r[1] = has_r1 ? r[0] + 1 : r[0];
      c[0] = 2 * cp;
      c[1] = has_c1 ? c[0] + 1 : c[0];
      valid = 0x1 | (has_c1 ? 0x2 : 0) | (has_r1 ? 0x4 : 0) | (has_r1 && has_c1 ? 0x8 : 0);
    }
    Item it;
    it.bz = __builtin_amdgcn_readfirstlane(bz);
    it.valid = __builtin_amdgcn_readfirstlane(valid);
    it.r2 = __builtin_amdgcn_readfirstlane(r2);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      it.r[u] = __builtin_amdgcn_readfirstlane(r[u]);
      it.c[u] = __builtin_amdgcn_readfirstlane(c[u]);
    }
    return it;
  };
  // k-step list of an item (GEMM-O: the union of the two token blocks' selected heads); returns the
  // number of slabs.  Called by all threads together, when nobody reads the previous list any more.
  // GEMM-O: the flags of an item's two token blocks, fetched by the first wavefront (lane = head, two
  // bits per group of 64 heads; up to 128 heads travel this way, more are read when the list is built).
  // Asked for at the top of the item before, so that the two dependent memory latencies (segment
  // offset, flag byte) pass behind that item's main loop.
  constexpr int kFetchedHeads = 128;
  int seg_bz = -1, seg_off = 0;
  auto fetch_flags = [&](const Item& item) -> uint32_t {
    uint32_t f = 0;
    if constexpr (kReduce) {
      const int n_slices = p.k / p.head_dim;
      if (wv == 0 && n_slices <= kFetchedHeads) {
        // (the segment offset of the batch entry is kept: one memory latency less on the way to the flags)
        if (item.bz != seg_bz) {
          seg_bz = item.bz;
          seg_off = p.sparse_info_indptr[item.bz];
        }
        const uint8_t* info = p.sparse_info + seg_off;
        const uint32_t base0 =
            static_cast<uint32_t>(p.num_text_tokens + item.r[0] * kTile) / p.sparse_q_size * p.num_heads;
        const uint32_t base1 =
            static_cast<uint32_t>(p.num_text_tokens + item.r[1] * kTile) / p.sparse_q_size * p.num_heads;
        const bool want1 = (item.valid & 0xC) != 0;
        const bool pick = p.flag == 0;  // final pass picks bit 1, cache pass bit 0
#pragma unroll
        for (int g = 0; g < kFetchedHeads / 64; ++g) {
          const int h = g * 64 + lane;
          if (h < n_slices) {
            const uint32_t s0 = flag_bit(info, base0 + h) == pick ? 1u : 0u;
            const uint32_t s1 = want1 && (flag_bit(info, base1 + h) == pick) ? 2u : 0u;
            f |= (s0 | s1) << (2 * g);
          }
        }
      }
    }
    return f;
  };
  auto build_steps = [&](const Item& item, uint32_t fetched) -> int {
    const int bz = item.bz, valid = item.valid;
    const int r[2] = {item.r[0], item.r[1]};
    int n_iter;
    if constexpr (kReduce) {
      if (wv == 0) {
        const uint8_t* info = p.sparse_info + p.sparse_info_indptr[bz];
        const uint32_t base0 =
            static_cast<uint32_t>(p.num_text_tokens + r[0] * kTile) / p.sparse_q_size * p.num_heads;
        const uint32_t base1 =
            static_cast<uint32_t>(p.num_text_tokens + r[1] * kTile) / p.sparse_q_size * p.num_heads;
        const bool want1 = (valid & 0xC) != 0;
        const bool pick = p.flag == 0;  // final pass picks bit 1, cache pass bit 0
        int count = 0;
        const int n_slices = p.k / p.head_dim;
        const bool have_fetched = n_slices <= kFetchedHeads;
        for (int h0 = 0; h0 < n_slices; h0 += 64) {
          const int h = h0 + lane;
          bool s0 = false, s1 = false;
          if (have_fetched) {
            const uint32_t two = fetched >> (2 * (h0 >> 6));
            s0 = (two & 1) != 0;
            s1 = (two & 2) != 0;
          } else if (h < n_slices) {
            s0 = flag_bit(info, base0 + h) == pick;
            s1 = want1 && (flag_bit(info, base1 + h) == pick);
          }
          const unsigned long long mask = __ballot(s0 || s1);
          if (s0 || s1)
            s_heads[count + __popcll(mask & ((1ull << lane) - 1ull))] = h | (s0 << 16) | (s1 << 17);
          count += __popcll(mask);
        }
        if (lane == 0) s_nsel = count;
      }
      __syncthreads();
      // slabs of a head slice: full 64-wide ones, then (head_dim % 64 == 32) one that reaches 32 back
      // into the slab before it and counts for its second half only (the first slice of the matrix
      // instead reaches forward and counts for its first half)
      const int iph = (p.head_dim + kBK - 1) / kBK;
      n_iter = __builtin_amdgcn_readfirstlane(s_nsel) * iph;
      if (n_iter > 0) {
        for (int i = tid; i < n_iter + 4; i += kThreads) {
          const int ii = i < n_iter ? i : n_iter - 1;
          const int hv = s_heads[ii / iph];
          const int k0 = (hv & 0xFFFF) * p.head_dim + (ii % iph) * kBK;
          int e = k0;
          if ((ii % iph) * kBK + kBK > p.head_dim) e = k0 >= 32 ? (k0 - 32) | kZeroFirst : k0 | kZeroSecond;
          s_step[i] = e | (hv & 0x30000);
        }
      }
      __syncthreads();
    } else {
      n_iter = (p.k + kBK - 1) / kBK;
    }

    return n_iter;
  };
  int n_iter = 0;
  // k offset of step it (steps past the end repeat the last one); GEMM-O: plus the select bits
  auto step_entry = [&](int it) -> int {
    if constexpr (kReduce) {
      return __builtin_amdgcn_readfirstlane(s_step[it]);  // uniform: the descriptor choice below stays scalar
    } else {
      // (K % 64 == 32: the last slab reaches 32 back and counts for its second half only)
      const int i = it < n_iter ? it : n_iter - 1;
      return (i + 1) * kBK <= p.k ? i * kBK | 0x30000 : (p.k - kBK) | kZeroFirst | 0x30000;
    }
  };
  // the same without making the list's value scalar (that needs the LDS read to have returned)
  auto step_entry_raw = [&](int it) -> int {
    if constexpr (kReduce) {
      return s_step[it];
    } else {
      return step_entry(it);
    }
  };
  // ---- operand tiles: buffer resource descriptors in scalar registers ----
  // The X descriptors end with the matrix, so rows past M read as zeros; a token block that does
  // not select a slab's head (GEMM-O) loads through an empty descriptor: zeros, no memory access.
  const __amdgpu_buffer_rsrc_t rsrc_none = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(xg), 0, 0, 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc[4] = {rsrc_none, rsrc_none, rsrc_none, rsrc_none};
  auto make_rsrc = [&](const Item& item) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int rows_left = min(p.m - item.r[u] * kTile, kTile);  // >= 1
      rsrc[u] = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<T*>(xg + (static_cast<int64_t>(item.bz) * p.m + static_cast<int64_t>(item.r[u]) * kTile) * p.k), 0,
          rows_left * p.k * 2, 0x00020000);
      rsrc[2 + u] = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<T*>(wg + static_cast<int64_t>(item.c[u]) * kTile * p.k), 0, kTile * p.k * 2, 0x00020000);
    }
    if constexpr (!kReduce) {
      if (item.valid & kColStrip) {  // a column strip's fourth tile is its third X tile
        const int rows_left = min(p.m - item.r2 * kTile, kTile);
        rsrc[3] = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<T*>(xg + (static_cast<int64_t>(item.bz) * p.m + static_cast<int64_t>(item.r2) * kTile) * p.k), 0,
            rows_left * p.k * 2, 0x00020000);
      }
    }
  };
  int ld_off[4];
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) ld_off[jj] = (32 * wv + 8 * jj + (lane >> 3)) * p.k * 2 + ld_chunk * 16;
  // Staging registers: piece j of a slab waits here between its global load and its LDS write.
  u32x4 stg[P];
  auto gload = [&](int j, int entry) {
    const int t = j >> 2;  // tiles 0, 1: X of token block 0, 1 (select bits 16, 17 of the entry); 2, 3: W
    const bool sel = t >= 2 || ((entry >> (16 + t)) & 1) != 0;
    stg[j] = __builtin_amdgcn_raw_buffer_load_b128(sel ? rsrc[t] : rsrc_none, ld_off[j & 3], (entry & 0xFFFF) * 2, 0);
  };
  // kHalf: only one half of a slab that reaches into its neighbour counts; the other half of the X
  // pieces is cleared on the way to LDS
  auto keep_of = [&](int entry) -> unsigned {
    return (entry & kZeroFirst) ? ~mask_first : ((entry & kZeroSecond) ? mask_first : 0xFFFFFFFFu);
  };
  auto lwrite = [&](int j, int stage, unsigned keep) {
    const int t = j >> 2;
    uint8_t* dst = smem + stage * kStageBytes + t * kUnitBytes + (32 * wv + 8 * (j & 3)) * kRowBytes + wr_off[j & 1];
    u32x4 v = stg[j];
    if constexpr (kHalf) {
      if (t != 2) v &= keep;  // (every tile that can hold X; a W tile cleared along with its X tile changes nothing)
    }
    *reinterpret_cast<u32x4*>(dst) = v;
  };

  // The first slab of an item is requested before the epilogue of the item before it, so that its
  // latency (and the list work above) hides behind the stores.
  // Work items of unequal length (GEMM-O: every item walks its own head list) let the workgroups of an
  // XCD drift apart when each strides through the queue in fixed steps, and items that run together
  // then no longer share tiles in L2.  Long GEMM-O launches therefore take their items from a cursor
  // per XCD: the items in flight are always neighbours in the queue.  One thread pops, an item ahead
  // (the value is needed at the top of the next item and waits in a register until then).
  bool popping = false;
  if constexpr (kReduce) popping = p.cursor != nullptr;
  int popped = 0;
  auto pop = [&]() {
    if (tid == 0) popped = per_xcd + atomicAdd(p.cursor + xcd, 1);  // (the first per_xcd items are dealt by slot)
  };
  if (popping) pop();
  int work = slot;
  bool have = work < q_len;
  Item cur{};
  if (have) {
    cur = decode_item(work);
    n_iter = build_steps(cur, fetch_flags(cur));
    make_rsrc(cur);
    if (n_iter > 0) {
      const int e0 = step_entry(0);
#pragma unroll
      for (int j = 0; j < P; ++j) gload(j, e0);
    }
  }
  while (have) {
    const int bz = cur.bz, valid = cur.valid;
    // (no indexing by a run-time value: the item has to stay in scalar registers)
    int out_r = wr ? cur.r[1] : cur.r[0], out_c = wc ? cur.c[1] : cur.c[0];
    bool my_valid = (valid >> (wr * 2 + wc)) & 1;
    int a_tile = 2 + wc, b_tile = wr;  // LDS tiles of this wavefront's W and X operands
    if constexpr (!kReduce) {
      if (valid & kColStrip) {
        out_r = wv == 0 ? cur.r[0] : wv == 1 ? cur.r[1] : cur.r2;
        out_c = cur.c[0];
        my_valid = wv < 3 && ((valid >> wv) & 1);
        a_tile = 2;
        b_tile = wv == 2 ? 3 : wv;
      }
    }
    // (the next item is looked up here, while no accumulator is live)
    int next_work = work + per_xcd;
    if (popping) {
      if (tid == 0) s_popped = popped;
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_s_barrier();
      next_work = __builtin_amdgcn_readfirstlane(s_popped);
      if (next_work < q_len) pop();  // for the item after the next
    }
    const bool have_next = next_work < q_len;
    Item nxt{};
    uint32_t nxt_flags = 0;
    if (have_next) {
      nxt = decode_item(next_work);
      nxt_flags = fetch_flags(nxt);
    }
    // every wavefront is done with the ring (the previous item's epilogue turned through it)
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();

    // ---- pipeline ----
    // Two slab buffers in LDS (stage it % 2 holds slab it) and one slab in flight in the staging
    // registers.  Iteration it: substeps 0..2 of slab it run while the last three quarters of the
    // pieces of slab it+1 go from the staging registers into the other stage and the same pieces of
    // slab it+2 are requested; one barrier (every wavefront has read all of slab it and written all of
    // slab it+1); substep 3 runs while the first operands of slab it+1 are read, the first quarter of
    // slab it+2 goes into stage it % 2 and that of slab it+3 is requested.  Every substep issues the
    // same mix (sixteen MFMAs, eight operand reads, four LDS writes, four global loads), so the memory
    // path sees an even stream and a load has a whole slab period to arrive.
    if (n_iter > 0) {
      const int e0 = step_entry(0), e1 = step_entry(1), e2 = step_entry(2);
      {
        const unsigned keep = keep_of(e0);
#pragma unroll
        for (int j = 0; j < P; ++j) lwrite(j, 0, keep);
      }
#pragma unroll
      for (int j = 0; j < P; ++j) gload(j, e1);
      {
        const unsigned keep = keep_of(e1);
#pragma unroll
        for (int j = 0; j < PS; ++j) lwrite(j, 1, keep);
      }
#pragma unroll
      for (int j = 0; j < PS; ++j) gload(j, e2);
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
    }

    // ---- next item: list work and the request for its first slab (every wavefront, once per item,
    // after its last use of the ring and of the step list, before the epilogue: the slab's latency
    // hides behind the stores). ----
    int next_iter = 0;
    auto ring_free = [&]() {
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_s_barrier();  // every wavefront is done with the ring and with the step list
    };
    auto prefetch_next = [&]() {
      if (have_next) {
        next_iter = build_steps(nxt, nxt_flags);
        make_rsrc(nxt);
        if (next_iter > 0) {
          const int saved = n_iter;
          n_iter = next_iter;  // (step_entry of the listless form clamps against it)
          const int e0 = step_entry(0);
          n_iter = saved;
#pragma unroll
          for (int j = 0; j < P; ++j) gload(j, e0);
        }
      }
    };
    // ---- accumulators (bias / cached partial are added in the epilogue) ----
    // acc[nt][mt][i]: n = n0 + nt*32 + (i/4)*8 + g*4 + i%4, m = m0 + mt*32 + l32
    const int m0 = out_r * kTile;
    const int n0 = out_c * kTile;
    f32x16 acc[NT][MT];
    if (!my_valid) {
      // This wavefront's unit does not exist in this quad (unflagged, or past the matrix edge): it
      // only moves its pieces and keeps the barrier sequence of the others.
      for (int it = 0; it < n_iter; ++it) {
        const int st = it & 1;
        const int en1 = step_entry(it + 1), en2 = step_entry(it + 2), en3 = step_entry(it + 3);
        const unsigned keep1 = keep_of(en1), keep2 = keep_of(en2);
#pragma unroll
        for (int j = PS; j < P; ++j) {
          lwrite(j, st ^ 1, keep1);
          gload(j, en2);
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int j = 0; j < PS; ++j) {
          lwrite(j, st, keep2);
          gload(j, en3);
        }
      }
      ring_free();
      prefetch_next();
    } else {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[nt][mt][i] = 0.f;
      if (n_iter > 0) {
        // LDS byte offsets of this wavefront's operand rows inside a stage
        const int a_base = a_tile * kUnitBytes + l32 * kRowBytes;  // W rows nt*32 + l32
        const int b_base = b_tile * kUnitBytes + l32 * kRowBytes;  // X rows mt*32 + l32
        x8 a[2][NT], b[2][MT];
        // operand read idx of substep sub of the slab in `stage` into register set sub & 1, in the order
        // the MFMAs need them: W rows 0, all X rows, W rows 1..3
        auto lread = [&](int stage, int sub, int idx) {
          const uint8_t* st = smem + stage * kStageBytes;
          const int x = rd_x ^ (sub << 5);
          if (idx == 0) {
            a[sub & 1][0] = *reinterpret_cast<const x8*>(st + a_base + x);
          } else if (idx <= MT) {
            b[sub & 1][idx - 1] = *reinterpret_cast<const x8*>(st + b_base + (idx - 1) * 32 * kRowBytes + x);
          } else {
            a[sub & 1][idx - MT] = *reinterpret_cast<const x8*>(st + a_base + (idx - MT) * 32 * kRowBytes + x);
          }
        };
        // one substep: the MFMAs of register set `set`; in their shadow the operand reads of substep
        // rsub of the slab in rstage, and pieces j0..j0+3: staged -> LDS stage wstage, then the same
        // pieces of the slab with entry `lentry` -> staging
        auto substep = [&](int set, int rstage, int rsub, int wstage, int j0, unsigned keep, int lentry) {
#pragma unroll
          for (int i = 0; i < NT * MT; ++i) {
            const int nt = i / MT, mt = i % MT;
            acc[nt][mt] = TT::mfma(a[set][nt], b[set][mt], acc[nt][mt]);
            if ((i & 1) == 0) lread(rstage, rsub, i >> 1);
            if ((i & 3) == 1) lwrite(j0 + (i >> 2), wstage, keep);
            if ((i & 3) == 3) gload(j0 + (i >> 2), lentry);
            __builtin_amdgcn_sched_barrier(0);
          }
        };
#pragma unroll
        for (int idx = 0; idx < NT + MT; ++idx) lread(0, 0, idx);
        // (the step entries of the next three slabs ride along in scalar registers; the fourth is
        // read from the list a slab ahead and becomes scalar after the wait the barrier needs anyway,
        // so the list costs no wait of its own)
        int en1 = step_entry(1), en2 = step_entry(2), en3 = step_entry(3);
        for (int it = 0; it < n_iter; ++it) {
          const int st = it & 1;
          const int en4_raw = step_entry_raw(it + 4);
          const unsigned keep1 = keep_of(en1), keep2 = keep_of(en2);
          substep(0, st, 1, st ^ 1, PS, keep1, en2);
          substep(1, st, 2, st ^ 1, 2 * PS, keep1, en2);
          substep(0, st, 3, st ^ 1, 3 * PS, keep1, en2);
          __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): my reads of slab it and my writes of slab it+1 are done
          __builtin_amdgcn_s_barrier();        // ... for every wavefront
          const int en4 = __builtin_amdgcn_readfirstlane(en4_raw);
          substep(1, st ^ 1, 0, st, 0, keep2, en3);
          en1 = en2;
          en2 = en3;
          en3 = en4;
        }
      }
      ring_free();
      // The request for the next item's first slab goes out before the epilogue and its data waits in
      // the staging registers, except where the epilogue adds a cached partial: its pieces need those
      // registers, so there the request follows the stores.
      if constexpr (!kPartial) prefetch_next();

    // ---- epilogue ----
    // In the accumulator layout a lane owns one output row and runs of four columns: written from
    // there, a store instruction is 64 scattered 8-byte pieces (measured: ~12 % of the FLUX-sized
    // launches; the bias matrix read the same way, as much again).  Each wavefront therefore turns
    // its block through its own quarter of the ring, 32 rows at a time in fp32, and adds the bias and
    // stores from a layout in which 32 consecutive lanes cover one row.
    {
      // (the lane index is made opaque: otherwise the per-lane address terms are computed once per
      // kernel, spilled, and every reload waits for the store before it)
      int ln = lane;
      asm volatile("" : "+v"(ln));
      const int col4 = ln & 31, rsub = ln >> 5, wl32 = ln & 31, wg = ln >> 5;
      uint8_t* const region0 = smem + wv * (kSmemBytes / 4);
      float bvec[4] = {0.f, 0.f, 0.f, 0.f};
      // Fused quantisation (GEMM-Q): a unit is one (token block, head) slab.  Its absmax is taken
      // over the final values (accumulator + bias, formed here in the accumulator layout without
      // being kept: the bias is added for good after the turn below); scale = absmax / 448 (1 for a
      // zero slab).
      float qscale = 1.f;
      if constexpr (kQuant) {
        {
          const bool has_vec = p.bias_kind == FO_BIAS_VECTOR;
          // all sixteen bias pieces requested before the first is used
          x4 bvs[NT * 4];
#pragma unroll
          for (int i = 0; i < NT * 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) bvs[i][j] = static_cast<T>(0.f);
          if (has_vec) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
              for (int i4 = 0; i4 < 4; ++i4)
                bvs[nt * 4 + i4] = *reinterpret_cast<const x4*>(static_cast<const T*>(p.bias) + n0 + nt * 32 +
                                                                i4 * 8 + wg * 4);
          }
          __builtin_amdgcn_sched_barrier(0);
          float amax = 0.f;
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
#pragma unroll
              for (int mt = 0; mt < MT; ++mt)
                if (m0 + mt * 32 + wl32 < p.m) {
#pragma unroll
                  for (int j = 0; j < 4; ++j) {
                    // (an opaque copy: otherwise the copies read out of the accumulator registers here
                    // are kept for the turn below, and spilled)
                    float v = acc[nt][mt][i4 * 4 + j];
                    asm volatile("" : "+v"(v));
                    amax = fmaxf(amax, fabsf(v + static_cast<float>(bvs[nt * 4 + i4][j])));
                  }
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // (quarter by quarter: taken together they do not fit the registers)
          }
#pragma unroll
          for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
          qscale = amax > 0.f ? amax / 448.0f : 1.0f;
          if (lane == 0)
            p.y_scale[static_cast<int64_t>(out_c) * p.scale_row_len + bz * p.n_row_tiles + out_r] = qscale;
        }
      }
      if (p.bias_kind == FO_BIAS_VECTOR) {
        const x4 bv = *reinterpret_cast<const x4*>(static_cast<const T*>(p.bias) + n0 + col4 * 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) bvec[j] = static_cast<float>(bv[j]);
      }
      // Output (and the cached partial, if there is one) go through buffer descriptors that end with the
      // matrix: rows past M are dropped (read as zeros) by the address unit, no lane is masked and no
      // row is tested.  A null output gets an empty descriptor.
      const int rows_out = min(p.m - m0, kTile);
      const int64_t row0 = static_cast<int64_t>(bz) * p.m + m0;
      auto out_rsrc = [&](const void* base, int elem_bytes) {
        return __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint8_t*>(static_cast<const uint8_t*>(base) + row0 * p.n * elem_bytes), 0,
            base ? rows_out * p.n * elem_bytes : 0, 0x00020000);
      };
      // 32 rows of the block.  kMatrix: a cached partial [B, M, N] of element type BiasT is added;
      // kOutF32: the output is fp32
      // (the cached partial of 32 rows: sixteen pieces, the four values this lane adds to each of its
      // rows, all in flight together while the rows turn through LDS.  Requesting the next 32 rows'
      // pieces earlier, in a second register set or piece by piece as the first set is consumed, was
      // measured: the compiler then spills 100-300 registers, some of them inside the main loop.)
      auto load_partial = [&](int mt, auto* bm) {
        using BiasVec = typename std::remove_reference<decltype(bm[0])>::type;
        constexpr int kBytes = sizeof(BiasVec) / 4;  // of one element
        const __amdgpu_buffer_rsrc_t rb = out_rsrc(p.bias, kBytes);
        const int el_off = n0 + col4 * 4 + rsub * p.n;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int row_off = (mt * 32 + 2 * i) * p.n * kBytes;
          if constexpr (kBytes == 4) {
            bm[i] = __builtin_bit_cast(BiasVec, __builtin_amdgcn_raw_buffer_load_b128(rb, el_off * 4, row_off, 0));
          } else {
            bm[i] = __builtin_bit_cast(BiasVec, __builtin_amdgcn_raw_buffer_load_b64(rb, el_off * 2, row_off, 0));
          }
        }
      };
      auto turn_half = [&](int mt, auto matrix_tag, auto* bm, auto f32_tag) {
        constexpr bool kMatrix = decltype(matrix_tag)::value, kOutF32 = decltype(f32_tag)::value;
        uint8_t* const region = region0 + (mt & 1) * (kSmemBytes / 8);
        // 16-byte chunk c of row r sits at chunk position c ^ r (rows are 512 bytes = 32 chunks)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            f32x4 v;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = acc[nt][mt][i4 * 4 + j];
            const int chunk = nt * 8 + i4 * 2 + wg;
            *reinterpret_cast<f32x4*>(region + wl32 * 512 + ((chunk ^ wl32) << 4)) = v;
          }
        // this lane's rows are mt*32 + rsub + 2*i, its columns n0 + col4*4 .. +3: a lane offset and a
        // scalar offset per row
        const int el_off = n0 + col4 * 4 + rsub * p.n;  // in elements, row mt*32 + rsub
        auto row_off = [&](int i, int elem_bytes) { return (mt * 32 + 2 * i) * p.n * elem_bytes; };
        if constexpr (kMatrix) load_partial(mt, bm);
        const __amdgpu_buffer_rsrc_t ry = out_rsrc(p.y, kOutF32 ? 4 : 2);
        // eight rows at a time are read back (two LDS latencies per turn) and biased, then stored
        f32x4 vals[8];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          if ((i & 7) == 0) {
#pragma unroll
            for (int k = 0; k < 8; ++k) {
              const int rk = (i + k) * 2 + rsub;
              vals[k] = *reinterpret_cast<const f32x4*>(region + rk * 512 + ((col4 ^ rk) << 4));
            }
            __builtin_amdgcn_sched_barrier(0);
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if constexpr (kMatrix) {
              vals[i & 7][j] += static_cast<float>(bm[i][j]);
            } else {
              vals[i & 7][j] += bvec[j];
            }
          }
          const f32x4 v = vals[i & 7];
          // (stored with the streaming hint, cache policy 2: the output is not read again by this launch
          // and should not push operand tiles out of the L2; 0.5-1.5 % at both sizes)
          if constexpr (kOutF32) {
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), ry, el_off * 4, row_off(i, 4), 2);
          } else {
            x4 out;
#pragma unroll
            for (int j = 0; j < 4; ++j) out[j] = static_cast<T>(v[j]);
            typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
            __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, out), ry, el_off * 2, row_off(i, 2), 2);
          }
          if constexpr (kQuant) {
            float f[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) f[j] = fminf(fmaxf(v[j] / qscale, -448.0f), 448.0f);
            unsigned w8 = 0;
            w8 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], w8, false);
            w8 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w8, true);
            __builtin_amdgcn_raw_buffer_store_b32(w8, out_rsrc(p.y8, 1), el_off, row_off(i, 1), 0);
            typedef __attribute__((ext_vector_type(2))) float f32x2;
            const f32x2 h0 = __builtin_amdgcn_cvt_pk_f32_fp8(w8, false);
            const f32x2 h1 = __builtin_amdgcn_cvt_pk_f32_fp8(w8, true);
            unsigned l8 = 0;
            l8 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0] - h0[0], f[1] - h0[1], l8, false);
            l8 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2] - h1[0], f[3] - h1[1], l8, true);
            __builtin_amdgcn_raw_buffer_store_b32(l8, out_rsrc(p.y8_lo, 1), el_off, row_off(i, 1), 0);  // (dropped if null)
          }
        }
      };
      auto turn_all = [&](auto matrix_tag, auto bias_tag, auto f32_tag) {
        using BiasT = decltype(bias_tag);
        using BiasVec = typename std::conditional<sizeof(BiasT) == 4, f32x4, x4>::type;
        BiasVec bm[16];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) turn_half(mt, matrix_tag, bm, f32_tag);
      };
      using std::false_type;
      using std::true_type;
      if constexpr (!kReduce) {
        turn_all(false_type{}, T{}, false_type{});  // GEMM-Q: bias vector or none, output in the activation type
      } else if constexpr (kPartial) {
        if (p.bias_f32) {
          if (p.y_f32) turn_all(true_type{}, 0.f, true_type{}); else turn_all(true_type{}, 0.f, false_type{});
        } else {
          if (p.y_f32) turn_all(true_type{}, T{}, true_type{}); else turn_all(true_type{}, T{}, false_type{});
        }
      } else {
        if (p.y_f32) turn_all(false_type{}, T{}, true_type{}); else turn_all(false_type{}, T{}, false_type{});
      }
    }
      if constexpr (kPartial) prefetch_next();
    }
    cur = nxt;
    n_iter = next_iter;
    work = next_work;
    have = have_next;
  }
}

ListGeom make_geom(int32_t batch, int32_t m, int32_t n) {
  ListGeom gm;
  gm.batch = batch;
  gm.n_row_tiles = (m + kTile - 1) / kTile;
  gm.n_col_tiles = n / kTile;
  gm.n_win = (gm.n_row_tiles + kWindow - 1) / kWindow;
  gm.n_cp = (gm.n_col_tiles + 1) / 2;
  return gm;
}

int64_t workspace_ints(const ListGeom& gm, int64_t* max_quads_out) {
  const int64_t n_wt = static_cast<int64_t>(gm.batch) * gm.n_win, n_cells = n_wt * gm.n_cp;
  const int64_t max_quads = n_cells * kWindow;  // a cell of 16 rows x 2 columns yields at most 16 quads
  if (max_quads_out) *max_quads_out = max_quads;
  return 16 + kQuadInts * max_quads;
}

template <typename T, bool kReduce, bool kHalf, bool kAux>
int launch_half(GemmParams& p, const ListGeom& gm, bool use_flags, void* workspace, hipStream_t stream) {
  // (the attribute belongs to the kernel's code object on one device: set once per device; the flags
  // are atomic because host threads may launch concurrently, and setting it twice is harmless)
  static std::atomic<bool> attr_set[64] = {};
  int dev = 0;
  FO_HIP_CALL(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64 || !attr_set[dev].load(std::memory_order_acquire)) {
    FO_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<T, kReduce, kHalf, kAux>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kSmemBytes));
    if (dev >= 0 && dev < 64) attr_set[dev].store(true, std::memory_order_release);
  }
  int64_t max_quads = 0;
  workspace_ints(gm, &max_quads);
  p.n_row_tiles = gm.n_row_tiles;
  p.n_col_tiles = gm.n_col_tiles;
  p.n_cp = gm.n_cp;
  p.n_win = gm.n_win;
  p.inline_cells = 0;
  int num_cu = fo_num_cu();
  if (num_cu <= 0) return fo::fail(FO_ERR_HIP, "gemm: no device");
  int64_t grid = (num_cu + kXcds - 1) / kXcds * kXcds;  // one persistent workgroup per CU
  const int64_t cap = (max_quads + kXcds - 1) / kXcds * kXcds;
  if (grid > cap) grid = cap;
  if (grid < kXcds) grid = kXcds;
  if (!use_flags) {
    // every unit is computed: no list, the kernel enumerates the quads itself
    p.quads = nullptr;
    p.qoff = nullptr;
    // (cursors pay off when a workgroup sees several items; short launches keep the fixed stride and
    // save the extra launch)
    const int64_t items = static_cast<int64_t>(gm.batch) * gm.n_cp *
                          (gm.n_row_tiles / kWindow * (kWindow / 2) + (gm.n_row_tiles % kWindow + 1) / 2);
    if (kReduce && p.cursor != nullptr && items >= 4 * grid) {
      gemm_cursor_clear_kernel<<<1, 16, 0, stream>>>(p.cursor);
      FO_CHECK_LAUNCH();
    } else {
      p.cursor = nullptr;
    }
    gemm_kernel<T, kReduce, kHalf, kAux><<<static_cast<unsigned>(grid), kThreads, kSmemBytes, stream>>>(p);
    FO_CHECK_LAUNCH();
    return FO_OK;
  }
  const int64_t n_cells = static_cast<int64_t>(gm.batch) * gm.n_win * gm.n_cp;
  if (!kReduce && n_cells <= kInlineCells) {
    // short launch: the kernel lists its quads itself (one launch less)
    p.quads = nullptr;
    p.qoff = nullptr;
    p.inline_cells = static_cast<int32_t>(n_cells);
    gemm_kernel<T, kReduce, kHalf, kAux><<<static_cast<unsigned>(grid), kThreads, kSmemBytes, stream>>>(p);
    FO_CHECK_LAUNCH();
    return FO_OK;
  }
  int32_t* qoff = static_cast<int32_t*>(workspace);
  int32_t* quads = qoff + 16;
  ListArgs la;
  la.sparse_info = p.sparse_info;
  la.sparse_info_indptr = p.sparse_info_indptr;
  la.use_flags = use_flags ? 1 : 0;
  la.sparse_q_size = p.sparse_q_size;
  la.num_heads = p.num_heads;
  la.head_dim = p.head_dim;
  la.num_text_tokens = p.num_text_tokens;
  gemm_quads_kernel<<<1, kListThreads, 0, stream>>>(la, gm, quads, qoff);
  FO_CHECK_LAUNCH();
  p.quads = quads;
  p.qoff = qoff;
  gemm_kernel<T, kReduce, kHalf, kAux><<<static_cast<unsigned>(grid), kThreads, kSmemBytes, stream>>>(p);
  FO_CHECK_LAUNCH();
  return FO_OK;
}

// kHalf: the k range is cut into slabs of 64 and some slab counts for one half only (GEMM-Q: K % 64 == 32;
// GEMM-O: head slices of width 32 mod 64)
template <typename T, bool kReduce>
int launch(GemmParams& p, const ListGeom& gm, bool use_flags, void* workspace, hipStream_t stream) {
  const bool half = (kReduce ? p.head_dim : p.k) % kBK != 0;
  // fused quantisation (GEMM-Q) and the cached partial (GEMM-O) get instantiations of their own, so
  // that the plain kernels do not carry their registers
  if (kReduce ? p.bias_kind == FO_BIAS_MATRIX : p.y8 != nullptr)
    return half ? launch_half<T, kReduce, true, true>(p, gm, use_flags, workspace, stream)
                : launch_half<T, kReduce, false, true>(p, gm, use_flags, workspace, stream);
  return half ? launch_half<T, kReduce, true, false>(p, gm, use_flags, workspace, stream)
              : launch_half<T, kReduce, false, false>(p, gm, use_flags, workspace, stream);
}

int check_common(const void* x, const void* w, void* y, int dtype, int32_t batch, int32_t m,
                 int32_t n, int32_t k, int32_t sparse_q_size, int32_t num_qo_heads,
                 void* workspace, int64_t workspace_bytes, bool needs_list) {
  FO_REQUIRE(dtype == FO_BF16 || dtype == FO_F16, "gemm: only bf16 / fp16 operands are supported");
  FO_REQUIRE(batch > 0 && m > 0 && n > 0 && k > 0, "gemm: bad shape");
  FO_REQUIRE(n % 128 == 0 && k % 32 == 0, "only support N %% 128 == 0, K %% 32 == 0 (got N=%d K=%d)",
             n, k);
  FO_REQUIRE(k >= kBK, "gemm: K = %d is below the 64 columns one operand slab holds", k);
  FO_REQUIRE(k <= 65536, "gemm: K = %d is above 65536 (a k-step entry keeps its k offset in 16 bits)", k);
  FO_REQUIRE(sparse_q_size > 0 && num_qo_heads > 0 && n % num_qo_heads == 0,
             "gemm: bad sparse_q_size / num_qo_heads");
  FO_REQUIRE(x && w && y, "gemm: null pointer");
  FO_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) |
               reinterpret_cast<uintptr_t>(y)) & 15) == 0,
             "gemm: x, w, y must be 16-byte aligned");
  const ListGeom gm = make_geom(batch, m, n);
  FO_REQUIRE(static_cast<int64_t>(batch) * gm.n_win * gm.n_cp < (int64_t(1) << 24), "gemm: too many tiles");
  const int64_t need = 4 * workspace_ints(gm, nullptr);
  if (!needs_list) return FO_OK;  // the workspace only holds the tile list
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15))
    return fo::fail(FO_ERR_WORKSPACE, "gemm: workspace of %lld bytes (16-byte aligned) required, got %lld",
                    static_cast<long long>(need), static_cast<long long>(workspace_bytes));
  return FO_OK;
}

}  // namespace

extern "C" int64_t fo_gemm_workspace_bytes(int32_t batch, int32_t m, int32_t n) {
  if (batch <= 0 || m <= 0 || n <= 0) return 0;
  return 4 * workspace_ints(make_geom(batch, m, n), nullptr);
}

namespace {
int gemm_q_impl(const void* x, const void* w, const void* bias, void* y, uint8_t* y8, uint8_t* y8_lo,
                float* y_scale, int dtype, int32_t batch, int32_t m, int32_t n, int32_t k, int32_t sparse_q_size,
                int32_t num_qo_heads, const uint8_t* sparse_info, const int32_t* sparse_info_indptr,
                int32_t num_text_tokens, int is_full, void* workspace, int64_t workspace_bytes,
                void* stream) {
  if (int rc = check_common(x, w, y8 ? static_cast<void*>(y8) : y, dtype, batch, m, n, k, sparse_q_size,
                            num_qo_heads, workspace, workspace_bytes, !is_full))
    return rc;
  FO_REQUIRE((reinterpret_cast<uintptr_t>(y) & 15) == 0, "gemm: x, w, y must be 16-byte aligned");
  FO_REQUIRE(is_full || (sparse_info && sparse_info_indptr),
             "gemm: sparse_info and sparse_info_indptr are required unless is_full");
  FO_REQUIRE(num_text_tokens >= 0, "gemm: negative num_text_tokens");
  FO_REQUIRE(!bias || (reinterpret_cast<uintptr_t>(bias) & 7) == 0, "gemm: bias must be 8-byte aligned");
  GemmParams p{};
  p.x = x; p.w = w; p.bias = bias; p.y = y;
  p.sparse_info = is_full ? nullptr : sparse_info;
  p.sparse_info_indptr = sparse_info_indptr;
  p.batch = batch; p.m = m; p.n = n; p.k = k;
  p.sparse_q_size = sparse_q_size; p.num_heads = num_qo_heads; p.head_dim = n / num_qo_heads;
  p.num_text_tokens = num_text_tokens;
  p.flag = is_full ? 1 : 0;
  p.bias_kind = bias ? FO_BIAS_VECTOR : FO_BIAS_NONE;
  const ListGeom gm = make_geom(batch, m, n);
  if (y8) {
    FO_REQUIRE(y_scale, "gemm_q_quant: y_scale is null");
    FO_REQUIRE(p.head_dim == kTile, "gemm_q_quant: head width %d is not supported (only 128)", p.head_dim);
    FO_REQUIRE((reinterpret_cast<uintptr_t>(y8) & 3) == 0 && (reinterpret_cast<uintptr_t>(y8_lo) & 3) == 0,
               "gemm_q_quant: y8 and y8_lo must be 4-byte aligned");
    p.y8 = y8;
    p.y8_lo = y8_lo;
    p.y_scale = y_scale;
    p.scale_row_len = batch * gm.n_row_tiles;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dtype == FO_BF16 ? launch<__bf16, false>(p, gm, !is_full, workspace, s)
                          : launch<_Float16, false>(p, gm, !is_full, workspace, s);
}
}  // namespace

extern "C" int fo_gemm_q(const void* x, const void* w, const void* bias, void* y, int dtype,
                         int32_t batch, int32_t m, int32_t n, int32_t k, int32_t sparse_q_size,
                         int32_t num_qo_heads, const uint8_t* sparse_info,
                         const int32_t* sparse_info_indptr, int32_t num_text_tokens, int is_full,
                         void* workspace, int64_t workspace_bytes, void* stream) {
  FO_REQUIRE(y, "gemm: null pointer");
  return gemm_q_impl(x, w, bias, y, nullptr, nullptr, nullptr, dtype, batch, m, n, k, sparse_q_size,
                     num_qo_heads, sparse_info, sparse_info_indptr, num_text_tokens, is_full, workspace,
                     workspace_bytes, stream);
}

extern "C" int fo_gemm_q_quant(const void* x, const void* w, const void* bias, void* y, uint8_t* y8,
                               uint8_t* y8_lo, float* y_scale, int dtype, int32_t batch, int32_t m, int32_t n,
                               int32_t k, int32_t sparse_q_size, int32_t num_qo_heads,
                               const uint8_t* sparse_info, const int32_t* sparse_info_indptr,
                               int32_t num_text_tokens, int is_full, void* workspace,
                               int64_t workspace_bytes, void* stream) {
  FO_REQUIRE(y8, "gemm_q_quant: y8 is null");
  return gemm_q_impl(x, w, bias, y, y8, y8_lo, y_scale, dtype, batch, m, n, k, sparse_q_size, num_qo_heads,
                     sparse_info, sparse_info_indptr, num_text_tokens, is_full, workspace,
                     workspace_bytes, stream);
}

extern "C" int fo_gemm_o(const void* x, const void* w, const void* bias, void* y, int dtype,
                         int bias_kind, int bias_dtype, int y_dtype, int32_t batch, int32_t m,
                         int32_t n, int32_t k, int32_t sparse_q_size, int32_t num_qo_heads,
                         const uint8_t* sparse_info, const int32_t* sparse_info_indptr,
                         int32_t num_text_tokens, int is_for_cached, void* workspace,
                         int64_t workspace_bytes, void* stream) {
  if (int rc = check_common(x, w, y, dtype, batch, m, n, k, sparse_q_size, num_qo_heads, workspace,
                            workspace_bytes, false))
    return rc;
  FO_REQUIRE(sparse_info && sparse_info_indptr, "gemm_reduction: sparse_info is required");
  FO_REQUIRE(num_text_tokens >= 0, "gemm: negative num_text_tokens");
  const int head_dim = n / num_qo_heads;
  FO_REQUIRE(head_dim % 32 == 0 && k % head_dim == 0 && k / head_dim <= kMaxHeads && k / 32 <= kMaxSteps,
             "gemm_reduction: head slice width %d must be a multiple of 32 and divide K=%d <= 65536",
             head_dim, k);
  FO_REQUIRE(bias_kind == FO_BIAS_NONE || bias_kind == FO_BIAS_VECTOR || bias_kind == FO_BIAS_MATRIX,
             "gemm_reduction: bad bias kind");
  FO_REQUIRE(bias_kind == FO_BIAS_NONE || bias, "gemm_reduction: bias pointer is null");
  FO_REQUIRE(bias_kind != FO_BIAS_VECTOR || bias_dtype == dtype,
             "gemm_reduction: a bias vector must have the activation dtype");
  FO_REQUIRE(bias_kind != FO_BIAS_MATRIX || bias_dtype == dtype || bias_dtype == FO_F32,
             "gemm_reduction: a bias matrix must have the activation dtype or fp32");
  FO_REQUIRE(y_dtype == dtype || y_dtype == FO_F32, "gemm_reduction: bad output dtype");
  FO_REQUIRE(!bias || (reinterpret_cast<uintptr_t>(bias) & 15) == 0,
             "gemm_reduction: bias must be 16-byte aligned");
  GemmParams p{};
  p.x = x; p.w = w; p.bias = bias_kind == FO_BIAS_NONE ? nullptr : bias; p.y = y;
  p.sparse_info = sparse_info; p.sparse_info_indptr = sparse_info_indptr;
  p.batch = batch; p.m = m; p.n = n; p.k = k;
  p.sparse_q_size = sparse_q_size; p.num_heads = num_qo_heads; p.head_dim = head_dim;
  p.num_text_tokens = num_text_tokens;
  p.flag = is_for_cached ? 1 : 0;
  p.bias_kind = bias_kind;
  p.bias_f32 = bias_dtype == FO_F32;
  p.y_f32 = y_dtype == FO_F32;
  // (optional workspace: room for the work-item cursors of a long launch)
  p.cursor = workspace != nullptr && workspace_bytes >= 64 && (reinterpret_cast<uintptr_t>(workspace) & 3) == 0
                 ? static_cast<int32_t*>(workspace)
                 : nullptr;
  const ListGeom gm = make_geom(batch, m, n);
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dtype == FO_BF16 ? launch<__bf16, true>(p, gm, false, workspace, s)
                          : launch<_Float16, true>(p, gm, false, workspace, s);
}
