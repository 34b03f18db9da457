// Ragged block-sparse FlashAttention prefill for gfx950 (MI355X), driven by a decoded work list.
//
// One workgroup = 8 wavefronts (512 lanes, two per SIMD) owns one work-list row = one (request,
// 128-row q-block, head).  Wavefront w serves q rows 32*(w%4)..+31 and kv group w/4: the row's
// 64-key tiles are dealt alternately to the two kv groups, each group keeps its own running
// (max, sum, O) state and the two states are merged through LDS when the row ends.  Two wavefronts
// per SIMD let one wavefront's softmax (VALU) run under the other's matrix products (MFMA);
// splitting a row over two kv groups halves its latency, which is what bounds the tail when there
// are only a few rows per CU.  LDS operand reads are issued in batches ahead of the MFMAs that
// consume them (one wavefront can start a 128-bit LDS read only every ~32 cycles).
// Only the kv blocks listed for the row are ever loaded; q-blocks that are not in the list are
// never visited, so their output bytes stay untouched.
//
// Everything is computed transposed so that no register shuffle sits between the two products:
//     S^T[kv, q] = K . Q^T        (A = K tile from LDS, B = Q kept in registers)
//     O^T[d, q] += V^T . P^T      (A = V^T via LDS transpose reads, B = P^T = exp2 of S^T, which
//                                  already has the B-operand layout)
// With v_mfma_f32_32x32x16 every lane holds one q column of S^T / O^T, so the online-softmax row
// statistics are per-lane scalars plus one exchange with lane^32.
//
// K/V tiles go global -> LDS directly (global_load_lds_dwordx4: no staging registers, the copy of
// the next tile runs under the current tile's math), two LDS stages per kv group, one barrier per
// tile.  A wavefront's 64 lanes land on 1 KB of consecutive LDS, so instead of padding the tile
// rows (256 B = 16 chunks of 16 B) are XOR-swizzled: row r keeps logical chunk c at position
// c ^ f(r), f(r) = ((r & 3) << 2) | ((r >> 2) & 3), applied on the global side of the copy.  That
// makes both the row-wise 128-bit K reads (16 consecutive rows, one chunk column) and the 4-row
// transpose reads of V (4 rows x 4 chunks) hit every bank exactly once.
//
// Work distribution: workgroups are persistent and pop rows from 8 queues (one per XCD, chosen by
// blockIdx % 8) that the decoder filled head by head, so one XCD's L2 serves a few heads' K/V; an
// idle XCD steals from its neighbours.  The last workgroup to finish resets the queue cursors.
//
// Numerics follow the reference kernel (include/flashomni/attention/prefill.cuh:759-962): base-2
// softmax p = exp2(s*c - m*c) with c = sm_scale*log2(e), P rounded to the activation type before
// P.V, masked logits and the initial running max are the finite -5e4 of
// include/flashomni/math.cuh:32, O = acc * rcp(d) with one round-to-nearest cast, a row with no kv
// block writes zeros and lse = -5e4, lse = log2(d) + m*c.  (The row sum d is accumulated from the
// fp32 p values; the reference sums the rounded ones.)
#include <type_traits>

#include "fo_common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(4))) int i32x4;

constexpr float kNegInf = -5e4f;  // finite "infinity" of the reference
constexpr int kThreads = 512;
constexpr int kGroupThreads = 256;
constexpr int kBlockQ = 128, kBlockKV = 128, kHeadDim = 128;
constexpr int kTileKV = 64;
constexpr int kRowBytes = 256;   // one K or V row of 128 16-bit elements, unpadded (swizzled)
constexpr int kRowBytes8 = 128;  // one fp8 K row
constexpr int kVBytes = kTileKV * kRowBytes;
// LDS geometry of one kv group: two stages of (K tile, V tile); K is 16-bit or fp8
template <bool kFp8>
struct Geom {
  static constexpr int kKBytes = kTileKV * (kFp8 ? kRowBytes8 : kRowBytes);
  static constexpr int kStageBytes = kKBytes + kVBytes;
  static constexpr int kGroupBytes = 2 * kStageBytes;
  static constexpr int kSmemBytes = 2 * kGroupBytes;
};
constexpr int kXcds = 8;
constexpr float kLazyLog2 = 8.0f;  // the running max is raised only past a 2^8 overshoot
// merge area (reuses the tile buffers): O^T of kv group 1, then its (m, d)
constexpr int kMergeOBytes = 4 * 16 * 64 * 16;
static_assert(kMergeOBytes + 4 * 64 * 8 <= Geom<true>::kSmemBytes, "merge area must fit");

struct FaParams {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  float* lse;
  const float* q_scale;
  const float* k_scale;
  int64_t q_sn, q_sh, k_sn, k_sh, v_sn, v_sh, o_sn, o_sh;
  const int32_t* qo_indptr;
  const int32_t* kv_indptr;
  const int32_t* q_blk_base;
  const int32_t* kv_blk_base;
  const int32_t* row_req;
  const int32_t* row_qb;
  const int32_t* row_head;
  const int32_t* kv_row_ptr;
  const int32_t* kv_idx;
  const int32_t* order;
  int32_t* sched;
  int32_t num_heads;
  int32_t n_q_blocks, n_kv_blocks;  // row lengths of q_scale / k_scale
  float sm_scale_log2;
};

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

typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void glb_void;

// chunk swizzle of a 256-byte LDS tile row r (16 chunks)
__device__ __forceinline__ int swz(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }
// chunk swizzle of a 128-byte LDS tile row r (8 chunks; two rows span the 64 banks)
__device__ __forceinline__ int swz8(int r) { return (r >> 1) & 7; }

// 64 lanes x 16 bytes, global -> LDS at lds_base + lane*16 (lds_base is wavefront-uniform)
__device__ __forceinline__ void copy16_to_lds(const void* gsrc, uint8_t* lds_base) {
  __builtin_amdgcn_global_load_lds((glb_void*)gsrc, (lds_void*)lds_base, 16, 0, 0);
}

// Four 16-bit values from a 4-row x 16-column LDS patch, transposed across a 16-lane group:
// the group's lane i (0..15) supplies the address of row i/4, columns 4*(i%4)..+3, and receives
// column i of rows 0..3.
__device__ __forceinline__ s16x4 lds_read_tr16(const uint8_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
}

// Pop the next row for this workgroup: own XCD queue first, then the neighbours'.
__device__ __forceinline__ int pop_row(const FaParams& p, int xcd) {
  for (int a = 0; a < kXcds; ++a) {
    const int x = (xcd + a) & (kXcds - 1);
    const int beg = p.sched[x], end = p.sched[x + 1];
    if (beg + __atomic_load_n(&p.sched[16 + x], __ATOMIC_RELAXED) >= end) continue;
    const int i = atomicAdd(&p.sched[16 + x], 1);
    if (beg + i < end) return p.order[beg + i];
  }
  return -1;
}

// T: element type of V, P and O (and of Q, K unless kFp8).  kFp8: Q and K are e4m3fn bytes with one
// dequantisation scale per (head, 128-token block); S^T then comes from
// v_mfma_scale_f32_32x32x64_f8f6f4 (64 d per instruction, unit block scale) and the two per-block
// scales are folded into the softmax scale of the tile.
template <typename T, bool kFp8>
__global__ void __launch_bounds__(kThreads) sparse_fa_kernel(const FaParams p) {
  using TT = Types<T>;
  using x8 = typename TT::x8;
  using x4 = typename TT::x4;
  using G = Geom<kFp8>;
  using TQK = typename std::conditional<kFp8, uint8_t, T>::type;
  constexpr int kStageBytes = G::kStageBytes, kKBytes = G::kKBytes, kGroupBytes = G::kGroupBytes;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  __shared__ int s_next_row;

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int qs = wv & 3, kg = wv >> 2;
  const int l32 = lane & 31, g = lane >> 5;
  const float c = p.sm_scale_log2;
  const TQK* __restrict__ qp = static_cast<const TQK*>(p.q);
  const TQK* __restrict__ kp = static_cast<const TQK*>(p.k);
  const T* __restrict__ vp = static_cast<const T*>(p.v);
  T* __restrict__ op = static_cast<T*>(p.o);
  uint8_t* const group_smem = smem + kg * kGroupBytes;

  // Copy assignment inside a kv group (4 wavefronts): copy instruction n = 4*j + qs, j = 0..3, fills
  // tile rows 4n..4n+3; this lane lands on row 4n + lane/16 at chunk position lane%16, so it must
  // fetch logical chunk (lane%16) ^ swz(row).  swz depends on row%16 = 4*qs + lane/16 only.
  const int cp_row = lane >> 4;
  const int cp_chunk = ((lane & 15) ^ swz(4 * qs + cp_row)) * 8;  // element offset inside the row
  // fp8 K tile (128-byte rows): copy instruction n = 4*j + qs, j = 0..1, fills rows 8n..8n+7; the
  // lane lands on row 8n + lane/8 at chunk position lane%8; swz8(row) = (4*(n%2) + lane/16) & 7
  const int cp8_row = lane >> 3;
  const int cp8_chunk = ((lane & 7) ^ ((4 * (qs & 1) + (lane >> 4)) & 7)) * 16;  // byte offset
  // K operand read: row mt*32 + l32, logical chunk 2*ks + g  ->  xor of a lane constant and ks<<5
  // (fp8: logical chunks 4*slab + 2*g and +1 of a 128-byte row)
  const int k_rd_base = l32 * (kFp8 ? kRowBytes8 : kRowBytes);
  const int k_rd_x = kFp8 ? ((2 * g) ^ swz8(l32)) << 4 : (g ^ swz(l32)) << 4;
  // V^T transpose read: this lane supplies row j = (lane%16)/4 of a 4-row patch that starts at kv
  // row 16*kk + 4*g (+8 for the second read), 8 bytes at element column 32*dt + 16*q2 + 4*(lane%4)
  int v_rd_off[4][2];
  {
    const int j = (lane & 15) >> 2, q2 = (lane >> 4) & 1, i4 = lane & 3;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int hi = 0; hi < 2; ++hi) {
        const int r = g * 4 + hi * 8 + j;
        const int chunk = dt * 4 + q2 * 2 + (i4 >> 1);
        v_rd_off[dt][hi] = r * kRowBytes + ((chunk ^ swz(r)) << 4) + (i4 & 1) * 8;
      }
  }

  for (;;) {
    __syncthreads();  // everyone is done with s_next_row and with the previous row's LDS data
    if (tid == 0) s_next_row = pop_row(p, blockIdx.x & (kXcds - 1));
    __syncthreads();
    const int w = s_next_row;
    if (w < 0) break;

    const int req = p.row_req[w], qb = p.row_qb[w], head = p.row_head[w];
    const int q_begin = p.qo_indptr[req] + qb * kBlockQ;
    const int q_rows = min(kBlockQ, p.qo_indptr[req + 1] - q_begin);
    const int kv_begin = p.kv_indptr[req];
    const int kv_len = p.kv_indptr[req + 1] - kv_begin;
    const int ptr0 = p.kv_row_ptr[w], nb = p.kv_row_ptr[w + 1] - ptr0;

    const int my_row = qs * 32 + l32;  // q row of this lane inside the block
    const bool row_ok = my_row < q_rows;
    const int64_t q_tok = q_begin + (row_ok ? my_row : q_rows - 1);

    if (nb == 0) {
      // listed row without kv blocks: zeros, lse = -5e4
      if (row_ok && kg == 0) {
        T* dst = op + q_tok * p.o_sn + static_cast<int64_t>(head) * p.o_sh + g * 64;
        const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < 8; ++j) reinterpret_cast<u32x4*>(dst)[j] = z;
        if (p.lse && g == 0) p.lse[q_tok * p.num_heads + head] = kNegInf;
      }
      continue;
    }

    // number of 64-key tiles; only the last listed block can be the request's ragged tail
    int n_tiles = 2 * nb;
    {
      const int last_blk = p.kv_idx[ptr0 + nb - 1];
      if (kv_len - last_blk * kBlockKV <= kTileKV) n_tiles -= 1;
    }
    const int my_tiles = (n_tiles - kg + 1) >> 1;  // tiles kg, kg+2, ...

    // Q operand: lane holds q row l32 of its q sub-tile, d = ks*16 + g*8 .. +7
    // (fp8: d = slab*64 + g*32 .. +31 for the two 64-wide slabs)
    x8 qreg[kFp8 ? 1 : 8];
    i32x8 qreg8[kFp8 ? 2 : 1];
    if constexpr (kFp8) {
      const uint8_t* src = qp + q_tok * p.q_sn + static_cast<int64_t>(head) * p.q_sh + g * 32;
#pragma unroll
      for (int sl = 0; sl < 2; ++sl) {
        const i32x4 lo = *reinterpret_cast<const i32x4*>(src + sl * 64);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(src + sl * 64 + 16);
        qreg8[sl] = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
    } else {
      const T* src = reinterpret_cast<const T*>(qp) + q_tok * p.q_sn + static_cast<int64_t>(head) * p.q_sh + g * 8;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) qreg[ks] = *reinterpret_cast<const x8*>(src + ks * 16);
    }
    // softmax scale in the log2 domain; with fp8 operands the per-block dequantisation scales of
    // q (one per row of the list) and k (one per kv block) are folded in tile by tile
    float cq = c;
    if constexpr (kFp8) cq *= p.q_scale[static_cast<int64_t>(head) * p.n_q_blocks + p.q_blk_base[req] + qb];
    const float* ksc = nullptr;
    if constexpr (kFp8) ksc = p.k_scale + static_cast<int64_t>(head) * p.n_kv_blocks + p.kv_blk_base[req];

    f32x16 o_acc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o_acc[dt][i] = 0.f;
    float m_run = kNegInf, d_part = 0.f;  // running max in the log2 domain (s * scale), partial sum
    float cs_next = cq;

    // Issue the global->LDS copy of this kv group's tile `it` into LDS stage it&1.
    const int64_t k_head = static_cast<int64_t>(head) * p.k_sh + (kFp8 ? cp8_chunk : cp_chunk);
    const int64_t v_head = static_cast<int64_t>(head) * p.v_sh + cp_chunk;
    auto copy_tile = [&](int it) {
      const int t = 2 * it + kg;
      const int blk = p.kv_idx[ptr0 + (t >> 1)];
      const int start = blk * kBlockKV + (t & 1) * kTileKV;
      const int valid = min(kTileKV, kv_len - start);
      const TQK* kt = kp + static_cast<int64_t>(kv_begin + start) * p.k_sn + k_head;
      const T* vt = vp + static_cast<int64_t>(kv_begin + start) * p.v_sn + v_head;
      uint8_t* kdst = group_smem + (it & 1) * kStageBytes;
      uint8_t* vdst = kdst + kKBytes;
      if constexpr (kFp8) cs_next = cq * ksc[blk];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = 4 * j + qs;
        int r = 4 * n + cp_row;
        r = r < valid ? r : valid - 1;  // ragged tail: re-read the last valid row, never overrun
        if constexpr (!kFp8) copy16_to_lds(kt + static_cast<int64_t>(r) * p.k_sn, kdst + n * 1024);
        copy16_to_lds(vt + static_cast<int64_t>(r) * p.v_sn, vdst + n * 1024);
      }
      if constexpr (kFp8) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int n = 4 * j + qs;
          int r = 8 * n + cp8_row;
          r = r < valid ? r : valid - 1;
          copy16_to_lds(kt + static_cast<int64_t>(r) * p.k_sn, kdst + n * 1024);
        }
      }
      return valid;
    };

    const int n_iter = (n_tiles + 1) >> 1;
    int valid_next = kTileKV;
    if (my_tiles > 0) valid_next = copy_tile(0);

    for (int it = 0; it < n_iter; ++it) {
      const uint8_t* ks_base = group_smem + (it & 1) * kStageBytes;
      const uint8_t* vs_base = ks_base + kKBytes;
      const bool active = it < my_tiles;
      const int valid = valid_next;
      const float cs = cs_next;  // softmax scale of this tile
      // this wavefront's copies of tile `it` have landed; after the barrier everyone's have, and
      // everyone has finished reading the other stage
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
      __syncthreads();
      if (!active) continue;  // (only the last iteration of kv group 1; no barrier follows)
      if (it + 1 < my_tiles) valid_next = copy_tile(it + 1);

      // ---- S^T = K . Q^T : two 32-key tiles x 32 q; all operand reads are issued up front ----
      f32x16 s[2];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[mt][i] = 0.f;
      if constexpr (kFp8) {
        i32x8 k8[2][2];  // [32-key tile][64-wide d slab]: 32 consecutive fp8 of row l32
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int sl = 0; sl < 2; ++sl) {
            const uint8_t* rowp = ks_base + mt * 32 * kRowBytes8 + k_rd_base;
            const i32x4 lo = *reinterpret_cast<const i32x4*>(rowp + (k_rd_x ^ (sl << 6)));
            const i32x4 hi = *reinterpret_cast<const i32x4*>(rowp + ((k_rd_x ^ (sl << 6)) ^ 16));
            k8[mt][sl] = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int sl = 0; sl < 2; ++sl)
            s[mt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(k8[mt][sl], qreg8[sl], s[mt], 0, 0, 0,
                                                                    0x7f7f7f7f, 0, 0x7f7f7f7f);
      } else {
        x8 ka[8], kb[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
          ka[ks] = *reinterpret_cast<const x8*>(ks_base + k_rd_base + (k_rd_x ^ (ks << 5)));
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
          kb[ks] = *reinterpret_cast<const x8*>(ks_base + 32 * kRowBytes + k_rd_base + (k_rd_x ^ (ks << 5)));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) s[0] = TT::mfma(ka[ks], qreg[ks], s[0]);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) s[1] = TT::mfma(kb[ks], qreg[ks], s[1]);
      }

      // all V^T operands of the tile (4 slabs of 16 keys x 4 d tiles): in flight during the
      // softmax, in the registers the K operands just vacated
      x8 vop[4][4];
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const uint8_t* base = vs_base + kk * 16 * kRowBytes;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
          union {
            s16x4 h[2];
            x8 v;
          } a;
          a.h[0] = lds_read_tr16(base + v_rd_off[dt][0]);
          a.h[1] = lds_read_tr16(base + v_rd_off[dt][1]);
          vop[kk][dt] = a.v;
        }
      }
      __builtin_amdgcn_sched_barrier(0);

      // ---- online softmax (per lane: one q column, 32 kv values), log2 domain: x = s * cs ----
      if (valid < kTileKV) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int kv = mt * 32 + (i >> 2) * 8 + g * 4 + (i & 3);
            if (kv >= valid) s[mt][i] = -INFINITY;  // p = 0 whatever the scale
          }
      }
      float mx = s[0][0];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[mt][i]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64)) * cs;
      // The running max is only raised when a row's new max exceeds it by more than kLazyLog2
      // (p then stays <= 2^kLazyLog2, harmless in fp32 / bf16 / fp16): the rescale of O leaves the
      // steady-state path.
      if (__builtin_expect(__any(mx - m_run > kLazyLog2), 0)) {
        const float m_new = fmaxf(m_run, mx);
        const float scale = __builtin_amdgcn_exp2f(m_run - m_new);
        d_part *= scale;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o_acc[dt][i] *= scale;
        m_run = m_new;
      }
      x8 pb[4];
      float psum = 0.f;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mt][i], cs, -m_run));
          psum += e;
          pb[mt * 2 + (i >> 3)][i & 7] = static_cast<T>(e);
        }
      d_part += psum;
      __builtin_amdgcn_sched_barrier(0);

      // ---- O^T += V^T . P^T : four 16-key slabs x four 32-wide d tiles ----
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) o_acc[dt] = TT::mfma(vop[kk][dt], pb[kk], o_acc[dt]);
    }

    // ---- merge the two kv groups through LDS, then write the row ----
    __syncthreads();  // all tile reads done: the tile buffers can be reused
    f32x4* mo = reinterpret_cast<f32x4*>(smem);
    float* md = reinterpret_cast<float*>(smem + kMergeOBytes);
    if (kg == 1) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          f32x4 t4;
#pragma unroll
          for (int j = 0; j < 4; ++j) t4[j] = o_acc[dt][i4 * 4 + j];
          mo[(qs * 16 + dt * 4 + i4) * 64 + lane] = t4;
        }
      md[(qs * 64 + lane) * 2 + 0] = m_run;
      md[(qs * 64 + lane) * 2 + 1] = d_part;
    }
    __syncthreads();
    if (kg == 0) {
      const float m1 = md[(qs * 64 + lane) * 2 + 0], d1 = md[(qs * 64 + lane) * 2 + 1];
      const float m = fmaxf(m_run, m1);
      const float a0 = __builtin_amdgcn_exp2f(m_run - m);
      const float a1 = __builtin_amdgcn_exp2f(m1 - m);
      const float d_lane = d_part * a0 + d1 * a1;
      const float d_tot = d_lane + __shfl_xor(d_lane, 32, 64);
      const float inv = __builtin_amdgcn_rcpf(d_tot);
      const float w0 = a0 * inv, w1 = a1 * inv;
      if (row_ok) {
        T* dst = op + q_tok * p.o_sn + static_cast<int64_t>(head) * p.o_sh;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            const f32x4 t4 = mo[(qs * 16 + dt * 4 + i4) * 64 + lane];
            x4 out;
#pragma unroll
            for (int j = 0; j < 4; ++j)
              out[j] = static_cast<T>(o_acc[dt][i4 * 4 + j] * w0 + t4[j] * w1);
            *reinterpret_cast<x4*>(dst + dt * 32 + i4 * 8 + g * 4) = out;
          }
        if (p.lse && g == 0)
          p.lse[q_tok * p.num_heads + head] = __builtin_amdgcn_logf(d_tot) + m;
      }
    }
  }

  // the last workgroup to leave rewinds the queues for the next launch
  if (tid == 0) {
    __threadfence();
    const int done = atomicAdd(&p.sched[24], 1);
    if (done == static_cast<int>(gridDim.x) - 1) {
      for (int x = 0; x < kXcds; ++x) p.sched[16 + x] = 0;
      p.sched[24] = 0;
    }
  }
}

template <typename T, bool kFp8>
int launch(const FaParams& p, int64_t max_rows, hipStream_t stream) {
  constexpr int kSmemBytes = Geom<kFp8>::kSmemBytes;
  static bool attr_set = false;
  if (!attr_set) {
    FO_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(&sparse_fa_kernel<T, kFp8>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kSmemBytes));
    attr_set = true;
  }
  int num_cu = fo_num_cu();
  if (num_cu <= 0) return fo::fail(FO_ERR_HIP, "sparse_fa: no device");
  int64_t grid = num_cu;  // one persistent workgroup per CU (LDS bound)
  if (grid > max_rows) grid = max_rows;
  sparse_fa_kernel<T, kFp8><<<static_cast<unsigned>(grid), kThreads, kSmemBytes, stream>>>(p);
  FO_CHECK_LAUNCH();
  return FO_OK;
}

}  // namespace

extern "C" int fo_sparse_fa_run(const void* q, const void* k, const void* v, void* o, float* lse,
                                int dtype, const float* q_scale, const float* k_scale,
                                int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n,
                                int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h,
                                int64_t o_stride_n, int64_t o_stride_h, const int32_t* qo_indptr,
                                const int32_t* kv_indptr, const int32_t* q_blk_base,
                                const int32_t* kv_blk_base, int32_t n_q_blocks,
                                int32_t n_kv_blocks, const int32_t* row_req,
                                const int32_t* row_qb, const int32_t* row_head,
                                const int32_t* kv_row_ptr, const int32_t* kv_idx,
                                const int32_t* order, int32_t* sched, int64_t max_rows,
                                int32_t num_heads, int32_t head_dim, int32_t block_q,
                                int32_t block_kv, float sm_scale, void* stream) {
  FO_REQUIRE(head_dim == kHeadDim, "sparse_fa: head_dim %d is not supported (only 128)", head_dim);
  FO_REQUIRE(block_q == kBlockQ && block_kv == kBlockKV,
             "sparse_fa: sparse block sizes (%d, %d) are not supported (only 128, 128)", block_q,
             block_kv);
  FO_REQUIRE(dtype == FO_BF16 || dtype == FO_F16 || dtype == FO_FP8_E4M3,
             "sparse_fa: unsupported dtype code %d", dtype);
  FO_REQUIRE(num_heads > 0 && max_rows >= 0, "sparse_fa: bad sizes");
  if (max_rows == 0) return FO_OK;
  FO_REQUIRE(q && k && v && o && qo_indptr && kv_indptr && row_req && row_qb && row_head &&
                 kv_row_ptr && kv_idx && order && sched,
             "sparse_fa: null pointer");
  const int64_t strides[8] = {q_stride_n, q_stride_h, k_stride_n, k_stride_h,
                              v_stride_n, v_stride_h, o_stride_n, o_stride_h};
  for (int i = 0; i < 8; ++i)
    FO_REQUIRE(strides[i] % (dtype == FO_FP8_E4M3 && i < 4 ? 16 : 8) == 0 && strides[i] > 0,
               "sparse_fa: strides must be positive multiples of 16 bytes (128-bit accesses)");
  if (dtype == FO_FP8_E4M3)
    FO_REQUIRE(q_scale && k_scale && q_blk_base && kv_blk_base && n_q_blocks > 0 && n_kv_blocks > 0,
               "sparse_fa: fp8 q/k need q_scale, k_scale, the block numbering and the scale row lengths");
  for (const void* ptr : {q, k, v, static_cast<const void*>(o)})
    FO_REQUIRE((reinterpret_cast<uintptr_t>(ptr) & 15) == 0,
               "sparse_fa: q/k/v/o must be 16-byte aligned");

  FaParams p;
  p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse;
  p.q_scale = q_scale; p.k_scale = k_scale;
  p.q_sn = q_stride_n; p.q_sh = q_stride_h; p.k_sn = k_stride_n; p.k_sh = k_stride_h;
  p.v_sn = v_stride_n; p.v_sh = v_stride_h; p.o_sn = o_stride_n; p.o_sh = o_stride_h;
  p.qo_indptr = qo_indptr; p.kv_indptr = kv_indptr;
  p.q_blk_base = q_blk_base; p.kv_blk_base = kv_blk_base;
  p.row_req = row_req; p.row_qb = row_qb; p.row_head = row_head;
  p.kv_row_ptr = kv_row_ptr; p.kv_idx = kv_idx; p.order = order; p.sched = sched;
  p.num_heads = num_heads; p.n_q_blocks = n_q_blocks; p.n_kv_blocks = n_kv_blocks;
  p.sm_scale_log2 = sm_scale * 1.44269504088896340736f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == FO_BF16) return launch<__bf16, false>(p, max_rows, s);
  if (dtype == FO_F16) return launch<_Float16, false>(p, max_rows, s);
  return launch<__bf16, true>(p, max_rows, s);
}
