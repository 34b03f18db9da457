// GEMM-Q and GEMM-O (with reduction) for gfx950: MFMA tile GEMMs that skip work according to the
// bit-packed (token-block, head) flags.
//
//   GEMM-Q  y[b, iy-tile, ix-tile] = x[b, iy-tile, :] . w[ix-tile, :]^T + bias   for flagged tiles;
//           the other tiles are never touched (reference: gemm/w16a16/gemm.cuh:50-58, 83-92).
//   GEMM-O  y[b, iy-tile, :] = init + sum_{selected heads h} x[:, h-slice] . w[:, h-slice]^T
//           where unselected head slices are never loaded
//           (reference: gemm/w16a16/gemm_reduction.cuh:77-95, 126-160).
//
// Tiling.  The skip flags have a 128 x 128 granularity, but a 128 x 128 workgroup tile with 64 x 64
// wavefront tiles needs one LDS operand read per MFMA, and LDS reads saturate before the matrix
// cores do.  So a workgroup (4 wavefronts, one per SIMD) computes a *pair* of flagged units that
// share one operand:
//   GEMM-Q: two flagged token blocks of the same head column (shared: the W tile)  -> 256 x 128
//   GEMM-O: two column blocks of the same token block (shared: the A tile)         -> 128 x 256
// Each wavefront owns a 128 x 64 piece (8 MFMA tiles of 32 x 32, 128 accumulators): six operand
// reads feed eight MFMAs.  A small kernel first compacts the GEMM-Q flags of every head column
// into the pair list (order inside the list is by column; the output does not depend on it).
//
// Data path.  BK = 64.  Operand tiles go global -> LDS directly (global_load_lds_dwordx4) into a
// 3-stage ring, two k steps ahead of the math, one barrier per k step.  A wavefront's copy lands
// on 1 KB of consecutive LDS (8 rows of 128 B), so rows are XOR-swizzled instead of padded: row r
// keeps logical 16-byte chunk c at position c ^ ((r >> 1) & 7), applied on the global side; the
// 128-bit operand reads of 16 consecutive rows then cover all 64 banks.
//
// The product is formed transposed (A operand = W rows, B operand = X rows) so that in the 32 x 32
// accumulator layout a lane owns one output row and runs of 4 consecutive columns: the epilogue
// reads the init matrix and writes the result with 8/16-byte accesses without going through LDS.
// fp32 accumulation starts from the init value converted to fp32; one round-to-nearest cast at
// the end.
//
// Work order.  Workgroups are persistent (one per CU).  The work is cut into windows of 16 token
// blocks; inside a window XCD x (= blockIdx % 8) takes the head columns congruent to x mod 8
// (GEMM-Q) / the x-th contiguous eighth of the (column pair, token block) entries (GEMM-O).  The
// ~32 workgroups of an XCD therefore work at the same time on a 16-token-block x few-column patch, whose operand tiles they share through that XCD's L2, and
// all XCDs sweep the token windows together, so the activations stream from HBM once while the
// weights stay in the memory-side cache.
#include "fo_common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void glb_void;

constexpr int kThreads = 256;
constexpr int kTile = 128;  // unit edge = granularity of the skip flags
constexpr int kBK = 64;
constexpr int kRowBytes = kBK * 2;                 // one LDS row: 64 elements, 8 chunks of 16 B
constexpr int kUnitBytes = kTile * kRowBytes;      // one 128-row operand tile: 16 KB
constexpr int kStageBytes = 3 * kUnitBytes;        // shared tile + two paired tiles
constexpr int kStages = 3;
constexpr int kSmemBytes = kStages * kStageBytes;  // 144 KB
constexpr int kCopiesPerWave = 3 * kUnitBytes / 1024 / 4;  // 12 copy instructions per stage
constexpr int kMaxHeads = 256;
constexpr int kXcds = 8;
constexpr int kPairThreads = 256;
constexpr int kPairScanThreads = 1024;
constexpr int kWindow = 16;  // token blocks per scheduling window

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
  const int32_t* pairs;  // GEMM-Q: int4 (b, ix, iy0, iy1) per pair, queue by queue
  const int32_t* qoff;   // GEMM-Q: qoff[0..8] queue boundaries inside `pairs`
  int32_t batch, m, n, k;
  int32_t sparse_q_size, num_heads, head_dim, num_text_tokens;
  int32_t flag;       // GEMM-Q: is_full.  GEMM-O: is_for_cached
  int32_t bias_kind;  // FO_BIAS_*
  int32_t bias_f32;   // matrix bias is fp32
  int32_t y_f32;      // output is fp32
};

// 64 lanes x 16 bytes, global -> LDS at lds_base + lane*16 (lds_base is wavefront-uniform)
__device__ __forceinline__ void copy16_to_lds(const void* gsrc, uint8_t* lds_base) {
  __builtin_amdgcn_global_load_lds((glb_void*)gsrc, (lds_void*)lds_base, 16, 0, 0);
}

__device__ __forceinline__ bool flag_bit(const uint8_t* info, uint32_t bit) {
  return (info[bit >> 3] >> (bit & 7)) & 1;
}

// ---------------------------------------------------------------------------------------------
// GEMM-Q pair list.  A cell = (batch, window of 16 token blocks, head column); its flagged token
// blocks are paired up (an odd one out is paired with -1).  Cells are laid out queue by queue
// (queue x = columns congruent to x mod 8), window-major inside a queue; qoff[0..8] delimit the
// queues.  One workgroup: every thread owns a contiguous range of cells in that order.
// ---------------------------------------------------------------------------------------------
struct PairGeom {
  int32_t batch, n_row_tiles, n_col_tiles, n_win, cols_per_q;
};

__device__ __forceinline__ uint32_t cell_mask(const PairGeom& gm, int64_t key,
                                              const uint8_t* __restrict__ sparse_info,
                                              const int32_t* __restrict__ sparse_info_indptr,
                                              int32_t sparse_q_size, int32_t num_heads,
                                              int32_t head_dim, int32_t num_text_tokens, int is_full,
                                              int* b_out, int* col_out, int* row0_out) {
  // key = ((x * batch + b) * n_win + w) * cols_per_q + ci,  column = ci*8 + x
  const int ci = static_cast<int>(key % gm.cols_per_q);
  int64_t t = key / gm.cols_per_q;
  const int w = static_cast<int>(t % gm.n_win);
  t /= gm.n_win;
  const int b = static_cast<int>(t % gm.batch);
  const int x = static_cast<int>(t / gm.batch);
  const int col = ci * kXcds + x;
  *b_out = b;
  *col_out = col;
  *row0_out = w * kWindow;
  if (col >= gm.n_col_tiles) return 0u;
  const int rows = min(kWindow, gm.n_row_tiles - w * kWindow);
  if (is_full) return (1u << rows) - 1u;
  const uint8_t* info = sparse_info + sparse_info_indptr[b];
  uint32_t mask = 0;
  for (int r = 0; r < rows; ++r) {
    const uint32_t bit = static_cast<uint32_t>(num_text_tokens + (w * kWindow + r) * kTile) / sparse_q_size *
                             num_heads + static_cast<uint32_t>(col * kTile) / head_dim;
    mask |= static_cast<uint32_t>(flag_bit(info, bit)) << r;
  }
  return mask;
}

__global__ void __launch_bounds__(kPairScanThreads) gemm_q_pairs_kernel(
    const uint8_t* __restrict__ sparse_info, const int32_t* __restrict__ sparse_info_indptr,
    PairGeom gm, int32_t sparse_q_size, int32_t num_heads, int32_t head_dim,
    int32_t num_text_tokens, int is_full, int32_t* __restrict__ pairs, int32_t* __restrict__ qoff) {
  __shared__ int32_t s_scan[kPairScanThreads];
  const int tid = threadIdx.x;
  const int64_t per_q = static_cast<int64_t>(gm.batch) * gm.n_win * gm.cols_per_q;
  const int64_t n_keys = per_q * kXcds;
  const int64_t chunk = (n_keys + kPairScanThreads - 1) / kPairScanThreads;
  const int64_t lo = tid * chunk, hi = lo + chunk < n_keys ? lo + chunk : n_keys;
  int b, col, row0;
  int32_t mine = 0;
  for (int64_t key = lo; key < hi; ++key)
    mine += (__popc(cell_mask(gm, key, sparse_info, sparse_info_indptr, sparse_q_size, num_heads, head_dim,
                              num_text_tokens, is_full, &b, &col, &row0)) + 1) >> 1;
  s_scan[tid] = mine;
  __syncthreads();
  for (int off = 1; off < kPairScanThreads; off <<= 1) {
    const int32_t v = tid >= off ? s_scan[tid - off] : 0;
    __syncthreads();
    s_scan[tid] += v;
    __syncthreads();
  }
  int32_t pos = s_scan[tid] - mine;
  if (tid == kPairScanThreads - 1) qoff[kXcds] = s_scan[tid];
  for (int64_t key = lo; key < hi; ++key) {
    if (key % per_q == 0) qoff[key / per_q] = pos;  // a queue starts here
    uint32_t mask = cell_mask(gm, key, sparse_info, sparse_info_indptr, sparse_q_size, num_heads, head_dim,
                              num_text_tokens, is_full, &b, &col, &row0);
    while (mask) {
      const int r0 = __ffs(mask) - 1;
      mask &= mask - 1;
      int r1 = -1;
      if (mask) {
        r1 = __ffs(mask) - 1;
        mask &= mask - 1;
      }
      int32_t* e = pairs + 4 * static_cast<int64_t>(pos++);
      e[0] = b;
      e[1] = col;
      e[2] = row0 + r0;
      e[3] = r1 < 0 ? -1 : row0 + r1;
    }
  }
  // queues past the last key range (possible when n_keys < threads) start at the total
  if (tid == 0 && n_keys == 0)
    for (int x = 0; x < kXcds; ++x) qoff[x] = 0;
}

// ---------------------------------------------------------------------------------------------
// Main kernel.  kReduce = false: GEMM-Q (pair = two token blocks, shared = W tile).
//               kReduce = true : GEMM-O (pair = two column blocks, shared = A tile).
// ---------------------------------------------------------------------------------------------
template <typename T, bool kReduce>
__global__ void __launch_bounds__(kThreads) gemm_kernel(const GemmParams p) {
  using TT = Types<T>;
  using x8 = typename TT::x8;
  using x4 = typename TT::x4;
  // accumulator tile of a wavefront, transposed product: NT n-tiles (W rows) x MT m-tiles (X rows)
  constexpr int NT = kReduce ? 4 : 2;
  constexpr int MT = kReduce ? 2 : 4;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  __shared__ int32_t s_heads[kMaxHeads];
  __shared__ int32_t s_nsel;

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int wp = wv >> 1, wh = wv & 1;  // which unit of the pair / which half of the shared side

  const T* __restrict__ xg = static_cast<const T*>(p.x);
  const T* __restrict__ wg = static_cast<const T*>(p.w);

  // copy assignment: per stage 48 copy instructions (n = 0..47), 8 LDS rows each; wavefront wv
  // issues n = 4*j + wv.  Instruction n fills rows 8*(n%16).. of tile n/16 (0 = shared, 1,2 = pair).
  // Lane i lands on row 8*(n%16) + i/8 at chunk position i%8 and must fetch logical chunk
  // (i%8) ^ ((row >> 1) & 7); (row >> 1) & 7 = (4*(n%2) + i/16) & 7 and n%2 = wv%2.
  const int cp_row = lane >> 3;
  const int cp_chunk = ((lane & 7) ^ ((4 * (wv & 1) + (lane >> 4)) & 7)) * 8;  // element offset
  // operand reads: row r = tile row base + l32, logical chunk 2*ks + g -> position ^ ((r >> 1) & 7)
  const int rd_x = (g ^ ((l32 >> 1) & 7)) << 4;  // xor-ed with ks << 5 at use; tile bases are
                                                 // multiples of 32 rows, so they do not change it

  // persistent work loop: XCD x (= blockIdx % 8) walks queue x, one entry per workgroup per round
  const int xcd = blockIdx.x & (kXcds - 1), slot = blockIdx.x >> 3;
  const int per_xcd = gridDim.x >> 3;  // host launches a multiple of 8 workgroups
  const int n_row_tiles = (p.m + kTile - 1) / kTile;
  int q_lo, q_len;  // GEMM-Q: range of `pairs`; GEMM-O: q_len entries, decoded in closed form
  // GEMM-O: a window holds rows x n_col_pairs entries in (column pair, token block) order and
  // XCD x owns the x-th contiguous eighth of every window
  const int n_col_pairs = (p.n / kTile + 1) / 2;
  const int full_w = n_row_tiles / kWindow, rem_rows = n_row_tiles % kWindow;
  const int chunk_full = kWindow * n_col_pairs / kXcds;  // 16 * P is a multiple of 8
  const int last_lo = rem_rows * n_col_pairs * xcd / kXcds;
  const int last_len = rem_rows * n_col_pairs * (xcd + 1) / kXcds - last_lo;
  const int per_b = full_w * chunk_full + last_len;
  if constexpr (kReduce) {
    q_lo = 0;
    q_len = p.batch * per_b;
  } else {
    q_lo = p.qoff[xcd];
    q_len = p.qoff[xcd + 1] - q_lo;
  }

  for (int work = slot; work < q_len; work += per_xcd) {
    // ---- decode the work item ----
    int bz, iy[2], ix[2];  // unit u of the pair is output tile (iy[u], ix[u]); -1 = absent
    if constexpr (kReduce) {
      bz = work / per_b;
      const int rem = work - bz * per_b;
      int wdw, idx, rows;
      if (rem < full_w * chunk_full) {
        wdw = rem / chunk_full;
        idx = xcd * chunk_full + (rem - wdw * chunk_full);
        rows = kWindow;
      } else {
        wdw = full_w;
        idx = last_lo + (rem - full_w * chunk_full);
        rows = rem_rows;
      }
      const int jp = idx / rows, rr = idx - jp * rows;
      iy[0] = iy[1] = wdw * kWindow + rr;
      ix[0] = 2 * jp;
      ix[1] = (2 * jp + 1) * kTile < p.n ? 2 * jp + 1 : -1;
    } else {
      const int32_t* e = p.pairs + 4 * static_cast<int64_t>(q_lo + work);
      bz = e[0];
      ix[0] = ix[1] = e[1];
      iy[0] = e[2];
      iy[1] = e[3];
      if (iy[1] < 0) ix[1] = -1;
    }
    const bool has2 = ix[1] >= 0;
    const bool my_valid = wp == 0 || has2;

    // ---- k-step list ----
    int n_iter;
    __syncthreads();  // previous work item: LDS tiles and s_heads are free
    if constexpr (kReduce) {
      if (wv == 0) {
        const uint8_t* info = p.sparse_info + p.sparse_info_indptr[bz];
        const uint32_t flag_base =
            static_cast<uint32_t>(p.num_text_tokens + iy[0] * kTile) / p.sparse_q_size * p.num_heads;
        int count = 0;
        const int n_slices = p.k / p.head_dim;
        for (int h0 = 0; h0 < n_slices; h0 += 64) {
          const int h = h0 + lane;
          bool sel = false;
          if (h < n_slices) {
            const bool one = flag_bit(info, flag_base + h);
            sel = p.flag ? !one : one;
          }
          const unsigned long long mask = __ballot(sel);
          if (sel) s_heads[count + __popcll(mask & ((1ull << lane) - 1ull))] = h;
          count += __popcll(mask);
        }
        if (lane == 0) s_nsel = count;
      }
      __syncthreads();
      n_iter = s_nsel * (p.head_dim / kBK);
    } else {
      n_iter = p.k / kBK;  // full k steps; a 32-wide K tail is finished after the loop
    }
    const int iters_per_head = kReduce ? p.head_dim / kBK : 1;
    auto k_of = [&](int it) -> int {
      if constexpr (kReduce) {
        return s_heads[it / iters_per_head] * p.head_dim + (it % iters_per_head) * kBK;
      } else {
        return it * kBK;
      }
    };

    // ---- global row pointers of the three operand tiles (tile 0 = shared, 1/2 = the pair) ----
    // GEMM-Q: shared = W rows of column ix, pair = X rows of token blocks iy[0], iy[1]
    // GEMM-O: shared = X rows of token block iy, pair = W rows of column blocks ix[0], ix[1]
    const T* tile_base[3];
    int tile_rows[3];  // valid rows (clamp for the M tail)
    {
      const T* xb = xg + static_cast<int64_t>(bz) * p.m * p.k;
      if constexpr (kReduce) {
        tile_base[0] = xb + static_cast<int64_t>(iy[0]) * kTile * p.k;
        tile_rows[0] = min(kTile, p.m - iy[0] * kTile);
        for (int u = 0; u < 2; ++u) {
          const int c = has2 || u == 0 ? ix[u] : ix[0];
          tile_base[1 + u] = wg + static_cast<int64_t>(c) * kTile * p.k;
          tile_rows[1 + u] = kTile;
        }
      } else {
        tile_base[0] = wg + static_cast<int64_t>(ix[0]) * kTile * p.k;
        tile_rows[0] = kTile;
        for (int u = 0; u < 2; ++u) {
          const int r = has2 || u == 0 ? iy[u] : iy[0];
          tile_base[1 + u] = xb + static_cast<int64_t>(r) * kTile * p.k;
          tile_rows[1 + u] = min(kTile, p.m - r * kTile);
        }
      }
    }
    auto copy_stage = [&](int it) {
      const int k0 = k_of(it);
      uint8_t* dst = smem + (it % kStages) * kStageBytes;
#pragma unroll
      for (int j = 0; j < kCopiesPerWave; ++j) {
        const int n = 4 * j + wv;         // 0..47
        const int tile = j >> 2;          // n / 16 (4*j + wv < 16 <=> j < 4)
        int r = 8 * (n & 15) + cp_row;
        r = r < tile_rows[tile] ? r : tile_rows[tile] - 1;
        copy16_to_lds(tile_base[tile] + static_cast<int64_t>(r) * p.k + k0 + cp_chunk, dst + n * 1024);
      }
    };

    // ---- accumulators, initialised from bias / cached partial ----
    // acc[nt][mt][i]: n = n0 + nt*32 + (i/4)*8 + g*4 + i%4, m = m0 + mt*32 + l32
    const int my_iy = kReduce ? iy[0] : iy[wp], my_ix = kReduce ? ix[wp] : ix[0];
    const int m0 = (my_valid ? my_iy : 0) * kTile + (kReduce ? wh * 64 : 0);
    const int n0 = (my_valid ? my_ix : 0) * kTile + (kReduce ? 0 : wh * 64);
    const int64_t y_batch = static_cast<int64_t>(bz) * p.m * p.n;
    f32x16 acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int mrow = m0 + mt * 32 + l32;
        const int mrow_c = mrow < p.m ? mrow : p.m - 1;
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          const int ncol = n0 + nt * 32 + i4 * 8 + g * 4;
          f32x4 init = {0.f, 0.f, 0.f, 0.f};
          if (p.bias_kind == FO_BIAS_VECTOR) {
            const x4 bv = *reinterpret_cast<const x4*>(static_cast<const T*>(p.bias) + ncol);
#pragma unroll
            for (int j = 0; j < 4; ++j) init[j] = static_cast<float>(bv[j]);
          } else if (p.bias_kind == FO_BIAS_MATRIX) {
            const int64_t off = y_batch + static_cast<int64_t>(mrow_c) * p.n + ncol;
            if (p.bias_f32) {
              init = *reinterpret_cast<const f32x4*>(static_cast<const float*>(p.bias) + off);
            } else {
              const x4 bv = *reinterpret_cast<const x4*>(static_cast<const T*>(p.bias) + off);
#pragma unroll
              for (int j = 0; j < 4; ++j) init[j] = static_cast<float>(bv[j]);
            }
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[nt][mt][i4 * 4 + j] = init[j];
        }
      }

    // LDS row bases of this wavefront's operands inside a stage
    // A operand (W rows): GEMM-Q shared tile rows wh*64.., GEMM-O pair tile wp rows 0..
    // B operand (X rows): GEMM-Q pair tile wp rows 0..,   GEMM-O shared tile rows wh*64..
    const int a_base = (kReduce ? (1 + wp) * kUnitBytes : wh * 64 * kRowBytes) + l32 * kRowBytes;
    const int b_base = (kReduce ? wh * 64 * kRowBytes : (1 + wp) * kUnitBytes) + l32 * kRowBytes;

    // ---- main loop: copies run two k steps ahead ----
    if (n_iter > 0) copy_stage(0);
    if (n_iter > 1) copy_stage(1);
    for (int it = 0; it < n_iter; ++it) {
      // tile `it` of this wavefront has landed (the 12 copies of tile it+1 may still be in flight)
      if (it + 1 < n_iter) {
        __builtin_amdgcn_s_waitcnt(0x0f70 | (kCopiesPerWave & 15));  // vmcnt(12)
      } else {
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
      }
      __syncthreads();  // everyone's copies of tile `it` landed; stage (it+2)%3 is no longer read
      if (it + 2 < n_iter) copy_stage(it + 2);
      // (a wavefront whose unit is absent computes on the duplicated tile and drops the result:
      // no branch in the loop body)
      const uint8_t* st = smem + (it % kStages) * kStageBytes;
      // operand registers are double-buffered: the reads of k step ks+1 are issued before the
      // MFMAs of k step ks (a single wavefront per SIMD has no other way to hide LDS latency)
      x8 a[2][NT], b[2][MT];
      auto load_ops = [&](int buf, int ks) {
        const int sw = rd_x ^ (ks << 5);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          a[buf][nt] = *reinterpret_cast<const x8*>(st + a_base + nt * 32 * kRowBytes + sw);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          b[buf][mt] = *reinterpret_cast<const x8*>(st + b_base + mt * 32 * kRowBytes + sw);
      };
      load_ops(0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < kBK / 16; ++ks) {
        if (ks + 1 < kBK / 16) load_ops((ks + 1) & 1, ks + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[nt][mt] = TT::mfma(a[ks & 1][nt], b[ks & 1][mt], acc[nt][mt]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // ---- 32-wide K tail (K % 64 == 32, GEMM-Q only): operands straight from global memory ----
    if (!kReduce && (p.k % kBK) != 0) {
      const int k0 = (p.k / kBK) * kBK;
      const int a_row0 = wh * 64, b_row0 = 0;  // rows inside the shared W tile / this unit's X tile
      const T* wsrc = tile_base[0];
      const T* xsrc = tile_base[1 + wp];
      const int xrows = tile_rows[1 + wp];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        x8 a[NT], b[MT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          a[nt] = *reinterpret_cast<const x8*>(wsrc + static_cast<int64_t>(a_row0 + nt * 32 + l32) * p.k +
                                               k0 + ks * 16 + g * 8);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          int r = b_row0 + mt * 32 + l32;
          r = r < xrows ? r : xrows - 1;
          b[mt] = *reinterpret_cast<const x8*>(xsrc + static_cast<int64_t>(r) * p.k + k0 + ks * 16 + g * 8);
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = TT::mfma(a[nt], b[mt], acc[nt][mt]);
      }
    }

    // ---- epilogue ----
    if (my_valid) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int mrow = m0 + mt * 32 + l32;
        if (mrow >= p.m) continue;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            const int ncol = n0 + nt * 32 + i4 * 8 + g * 4;
            const int64_t off = y_batch + static_cast<int64_t>(mrow) * p.n + ncol;
            if (p.y_f32) {
              f32x4 out;
#pragma unroll
              for (int j = 0; j < 4; ++j) out[j] = acc[nt][mt][i4 * 4 + j];
              *reinterpret_cast<f32x4*>(static_cast<float*>(p.y) + off) = out;
            } else {
              x4 out;
#pragma unroll
              for (int j = 0; j < 4; ++j) out[j] = static_cast<T>(acc[nt][mt][i4 * 4 + j]);
              *reinterpret_cast<x4*>(static_cast<T*>(p.y) + off) = out;
            }
          }
      }
    }
  }
}

template <typename T, bool kReduce>
int launch(const GemmParams& p, int64_t max_work, hipStream_t stream) {
  static bool attr_set = false;
  if (!attr_set) {
    FO_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<T, kReduce>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kSmemBytes));
    attr_set = true;
  }
  int num_cu = fo_num_cu();
  if (num_cu <= 0) return fo::fail(FO_ERR_HIP, "gemm: no device");
  int64_t grid = (num_cu + kXcds - 1) / kXcds * kXcds;  // one persistent workgroup per CU
  const int64_t cap = (max_work + kXcds - 1) / kXcds * kXcds;
  if (grid > cap) grid = cap;
  if (grid < kXcds) grid = kXcds;
  gemm_kernel<T, kReduce><<<static_cast<unsigned>(grid), kThreads, kSmemBytes, stream>>>(p);
  FO_CHECK_LAUNCH();
  return FO_OK;
}

int check_common(const void* x, const void* w, void* y, int dtype, int32_t batch, int32_t m,
                 int32_t n, int32_t k, int32_t sparse_q_size, int32_t num_qo_heads) {
  FO_REQUIRE(dtype == FO_BF16 || dtype == FO_F16, "gemm: only bf16 / fp16 operands are supported");
  FO_REQUIRE(batch > 0 && m > 0 && n > 0 && k > 0, "gemm: bad shape");
  FO_REQUIRE(n % 128 == 0 && k % 32 == 0, "only support N %% 128 == 0, K %% 32 == 0 (got N=%d K=%d)",
             n, k);
  FO_REQUIRE(sparse_q_size > 0 && num_qo_heads > 0 && n % num_qo_heads == 0,
             "gemm: bad sparse_q_size / num_qo_heads");
  FO_REQUIRE(x && w && y, "gemm: null pointer");
  FO_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) |
               reinterpret_cast<uintptr_t>(y)) & 15) == 0,
             "gemm: x, w, y must be 16-byte aligned");
  FO_REQUIRE(static_cast<int64_t>(batch) * ((m + kTile - 1) / kTile) * (n / kTile) < (int64_t(1) << 30),
             "gemm: too many tiles");
  return FO_OK;
}

}  // namespace

extern "C" int64_t fo_gemm_q_workspace_bytes(int32_t batch, int32_t m, int32_t n) {
  if (batch <= 0 || m <= 0 || n <= 0) return 0;
  const int64_t n_row_tiles = (m + kTile - 1) / kTile, n_win = (n_row_tiles + kWindow - 1) / kWindow;
  const int64_t max_pairs = static_cast<int64_t>(batch) * (n / kTile) * n_win * (kWindow / 2);
  return 64 + 16 * max_pairs;
}

extern "C" int fo_gemm_q(const void* x, const void* w, const void* bias, void* y, int dtype,
                         int32_t batch, int32_t m, int32_t n, int32_t k, int32_t sparse_q_size,
                         int32_t num_qo_heads, const uint8_t* sparse_info,
                         const int32_t* sparse_info_indptr, int32_t num_text_tokens, int is_full,
                         void* workspace, int64_t workspace_bytes, void* stream) {
  if (int rc = check_common(x, w, y, dtype, batch, m, n, k, sparse_q_size, num_qo_heads)) return rc;
  FO_REQUIRE(is_full || (sparse_info && sparse_info_indptr),
             "gemm: sparse_info and sparse_info_indptr are required unless is_full");
  FO_REQUIRE(num_text_tokens >= 0, "gemm: negative num_text_tokens");
  FO_REQUIRE(!bias || (reinterpret_cast<uintptr_t>(bias) & 7) == 0, "gemm: bias must be 8-byte aligned");
  const int64_t need = fo_gemm_q_workspace_bytes(batch, m, n);
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15))
    return fo::fail(FO_ERR_WORKSPACE, "gemm: workspace of %lld bytes (16-byte aligned) required, got %lld",
                    static_cast<long long>(need), static_cast<long long>(workspace_bytes));
  hipStream_t s = static_cast<hipStream_t>(stream);
  int32_t* qoff = static_cast<int32_t*>(workspace);
  int32_t* pairs = qoff + 16;
  PairGeom gm;
  gm.batch = batch;
  gm.n_row_tiles = (m + kTile - 1) / kTile;
  gm.n_col_tiles = n / kTile;
  gm.n_win = (gm.n_row_tiles + kWindow - 1) / kWindow;
  gm.cols_per_q = (gm.n_col_tiles + kXcds - 1) / kXcds;
  gemm_q_pairs_kernel<<<1, kPairScanThreads, 0, s>>>(is_full ? nullptr : sparse_info, sparse_info_indptr, gm,
                                                     sparse_q_size, num_qo_heads, n / num_qo_heads,
                                                     num_text_tokens, is_full ? 1 : 0, pairs, qoff);
  FO_CHECK_LAUNCH();
  GemmParams p{};
  p.x = x; p.w = w; p.bias = bias; p.y = y;
  p.sparse_info = is_full ? nullptr : sparse_info;
  p.sparse_info_indptr = sparse_info_indptr;
  p.pairs = pairs; p.qoff = qoff;
  p.batch = batch; p.m = m; p.n = n; p.k = k;
  p.sparse_q_size = sparse_q_size; p.num_heads = num_qo_heads; p.head_dim = n / num_qo_heads;
  p.num_text_tokens = num_text_tokens;
  p.flag = is_full ? 1 : 0;
  p.bias_kind = bias ? FO_BIAS_VECTOR : FO_BIAS_NONE;
  const int64_t max_pairs = static_cast<int64_t>(batch) * gm.n_col_tiles * gm.n_win * (kWindow / 2);
  return dtype == FO_BF16 ? launch<__bf16, false>(p, max_pairs, s) : launch<_Float16, false>(p, max_pairs, s);
}

extern "C" int fo_gemm_o(const void* x, const void* w, const void* bias, void* y, int dtype,
                         int bias_kind, int bias_dtype, int y_dtype, int32_t batch, int32_t m,
                         int32_t n, int32_t k, int32_t sparse_q_size, int32_t num_qo_heads,
                         const uint8_t* sparse_info, const int32_t* sparse_info_indptr,
                         int32_t num_text_tokens, int is_for_cached, void* stream) {
  if (int rc = check_common(x, w, y, dtype, batch, m, n, k, sparse_q_size, num_qo_heads)) return rc;
  FO_REQUIRE(sparse_info && sparse_info_indptr, "gemm_reduction: sparse_info is required");
  FO_REQUIRE(num_text_tokens >= 0, "gemm: negative num_text_tokens");
  const int head_dim = n / num_qo_heads;
  FO_REQUIRE(head_dim % kBK == 0 && k % head_dim == 0 && k / head_dim <= kMaxHeads,
             "gemm_reduction: head slice width %d must be a multiple of 64 and divide K=%d", head_dim, k);
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
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t work = static_cast<int64_t>(batch) * ((m + kTile - 1) / kTile) * ((n / kTile + 1) / 2);
  return dtype == FO_BF16 ? launch<__bf16, true>(p, work, s) : launch<_Float16, true>(p, work, s);
}
