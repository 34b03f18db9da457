// Ragged block-sparse FlashAttention prefill for gfx950 (MI355X), driven by a decoded work list.
//
// One workgroup (4 wavefronts of 64 lanes) owns one work-list row = one (request, 128-row q-block,
// head); each wavefront owns 32 q rows.  Only the kv blocks listed for the row are ever loaded;
// q-blocks that are not in the list are never visited, so their output bytes stay untouched.
//
// Everything is computed transposed so that no register shuffle sits between the two matrix
// products:   S^T[kv, q] = K . Q^T        (A = K tile from LDS, B = Q kept in registers)
//             O^T[d, q] += V^T . P^T      (A = V^T via LDS transpose reads, B = P^T = exp2 of S^T,
//                                          which is already in B-operand layout)
// With v_mfma_f32_32x32x16 every lane holds one q column of S^T / O^T, so the online-softmax row
// statistics are per-lane scalars plus one exchange with lane^32.
//
// K/V tiles of 64 kv rows are staged global -> registers -> LDS (128-bit accesses) in two LDS
// stages, one barrier per tile; LDS rows are padded (K: 272 B, V: 320 B) so that the 128-bit
// row-wise K reads and the 4-row transpose reads of V spread over all 64 banks.
//
// Numerics follow the reference kernel (include/flashomni/attention/prefill.cuh:759-962):
// base-2 softmax p = exp2(s*c - m*c) with c = sm_scale*log2(e), P rounded to the activation type
// before P.V and before the row sum, masked logits and the initial running max are the finite
// -5e4 of include/flashomni/math.cuh:32, O = acc * rcp(d) with one round-to-nearest cast, a row
// with no kv block writes zeros and lse = -5e4, lse = log2(d) + m*c.
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

constexpr float kNegInf = -5e4f;  // finite "infinity" of the reference
constexpr int kThreads = 256;
constexpr int kBlockQ = 128, kBlockKV = 128, kHeadDim = 128;
constexpr int kTileKV = 64;
constexpr int kKStride = 272;  // bytes per K row in LDS (256 + 16 pad)
constexpr int kVStride = 320;  // bytes per V row in LDS (256 + 64 pad)
constexpr int kKBytes = kTileKV * kKStride;
constexpr int kVBytes = kTileKV * kVStride;
constexpr int kStageBytes = kKBytes + kVBytes;
constexpr int kSmemBytes = 2 * kStageBytes;

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
  const int32_t* counts;
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

// Four 16-bit values from a 4-row x 16-column LDS patch, transposed across a 16-lane group:
// the group's lane i (0..15) supplies the address of row i/4, columns 4*(i%4)..+3, and receives
// column i of rows 0..3.
__device__ __forceinline__ s16x4 lds_read_tr16(const uint8_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
}

template <typename T>
__global__ void __launch_bounds__(kThreads, 2) sparse_fa_kernel(const FaParams p) {
  using TT = Types<T>;
  using x8 = typename TT::x8;
  using x4 = typename TT::x4;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int n_rows = p.counts[0];
  const float c = p.sm_scale_log2;
  const T* __restrict__ qp = static_cast<const T*>(p.q);
  const T* __restrict__ kp = static_cast<const T*>(p.k);
  const T* __restrict__ vp = static_cast<const T*>(p.v);
  T* __restrict__ op = static_cast<T*>(p.o);

  // staging assignment: chunk cc = tid + 256*i -> tile row cc/16, 16-byte column cc%16
  const int st_row = tid >> 4, st_col = tid & 15;

  for (int w = blockIdx.x; w < n_rows; w += gridDim.x) {
    const int req = p.row_req[w], qb = p.row_qb[w], head = p.row_head[w];
    const int q_begin = p.qo_indptr[req] + qb * kBlockQ;
    const int q_rows = min(kBlockQ, p.qo_indptr[req + 1] - q_begin);
    const int kv_begin = p.kv_indptr[req];
    const int kv_len = p.kv_indptr[req + 1] - kv_begin;
    const int ptr0 = p.kv_row_ptr[w], nb = p.kv_row_ptr[w + 1] - ptr0;

    const int my_row = wv * 32 + l32;  // q row of this lane inside the block
    const bool row_ok = my_row < q_rows;
    const int64_t q_tok = q_begin + (row_ok ? my_row : q_rows - 1);

    if (nb == 0) {
      // listed row without kv blocks: zeros, lse = -5e4
      if (row_ok) {
        T* dst = op + q_tok * p.o_sn + static_cast<int64_t>(head) * p.o_sh + g * 64;
        const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < 8; ++j) reinterpret_cast<u32x4*>(dst)[j] = z;
        if (p.lse && g == 0) p.lse[q_tok * p.num_heads + head] = kNegInf;
      }
      continue;
    }

    // number of 64-row tiles; only the last listed block can be the request's ragged tail
    int n_tiles = 2 * nb;
    {
      const int last_blk = p.kv_idx[ptr0 + nb - 1];
      if (kv_len - last_blk * kBlockKV <= kTileKV) n_tiles -= 1;
    }

    // Q operand: lane holds q row l32 of its wave, d = ks*16 + g*8 .. +7
    x8 qreg[8];
    {
      const T* src = qp + q_tok * p.q_sn + static_cast<int64_t>(head) * p.q_sh + g * 8;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) qreg[ks] = *reinterpret_cast<const x8*>(src + ks * 16);
    }

    f32x16 o_acc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o_acc[dt][i] = 0.f;
    float m_run = kNegInf, d_part = 0.f;

    u32x4 kst[4], vst[4];
    auto load_tile = [&](int t) {
      const int blk = p.kv_idx[ptr0 + (t >> 1)];
      const int start = blk * kBlockKV + (t & 1) * kTileKV;
      const int valid = min(kTileKV, kv_len - start);
      const int64_t head_k = static_cast<int64_t>(head) * p.k_sh + st_col * 8;
      const int64_t head_v = static_cast<int64_t>(head) * p.v_sh + st_col * 8;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int r = st_row + 16 * i;
        r = r < valid ? r : valid - 1;
        const int64_t tok = kv_begin + start + r;
        kst[i] = *reinterpret_cast<const u32x4*>(kp + tok * p.k_sn + head_k);
        vst[i] = *reinterpret_cast<const u32x4*>(vp + tok * p.v_sn + head_v);
      }
      return valid;
    };

    __syncthreads();  // previous row's LDS reads are complete
    int valid_next = load_tile(0);

    for (int t = 0; t < n_tiles; ++t) {
      uint8_t* ks_base = smem + (t & 1) * kStageBytes;
      uint8_t* vs_base = ks_base + kKBytes;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = st_row + 16 * i;
        *reinterpret_cast<u32x4*>(ks_base + r * kKStride + st_col * 16) = kst[i];
        *reinterpret_cast<u32x4*>(vs_base + r * kVStride + st_col * 16) = vst[i];
      }
      const int valid = valid_next;
      __syncthreads();
      if (t + 1 < n_tiles) valid_next = load_tile(t + 1);

      // ---- S^T = K . Q^T : 2 kv tiles of 32 x 32 q ----
      f32x16 s[2];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[mt][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          const x8 a = *reinterpret_cast<const x8*>(ks_base + (mt * 32 + l32) * kKStride +
                                                    ks * 32 + g * 16);
          s[mt] = TT::mfma(a, qreg[ks], s[mt]);
        }
      }

      // ---- online softmax (per lane: one q column, 32 kv values) ----
      if (valid < kTileKV) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int kv = mt * 32 + (i >> 2) * 8 + g * 4 + (i & 3);
            if (kv >= valid) s[mt][i] = kNegInf;
          }
      }
      float mx = s[0][0];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[mt][i]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run, mx);
      const float scale = __builtin_amdgcn_exp2f((m_run - m_new) * c);
      const float mc = m_new * c;
      m_run = m_new;

      x8 pb[4];
      float psum = 0.f;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mt][i], c, -mc));
          const T r = static_cast<T>(e);
          pb[mt * 2 + (i >> 3)][i & 7] = r;
          psum += static_cast<float>(r);
        }
      d_part = d_part * scale + psum;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[dt][i] *= scale;

      // ---- O^T += V^T . P^T ----
      // lane's transpose-read source: row (lane%16)/4 of the 4-row patch, columns 4*(lane%4)..
      const int tr_row = (lane & 15) >> 2;
      const int tr_col = ((lane >> 4) & 1) * 16 + (lane & 3) * 4;  // element column inside a d tile
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {     // 16-row kv slabs
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {   // 32-column d tiles
          const uint8_t* base = vs_base + (kk * 16 + g * 4 + tr_row) * kVStride +
                                (dt * 32 + tr_col) * 2;
          const s16x4 lo = lds_read_tr16(base);
          const s16x4 hi = lds_read_tr16(base + 8 * kVStride);
          union {
            s16x4 h[2];
            x8 v;
          } a;
          a.h[0] = lo;
          a.h[1] = hi;
          o_acc[dt] = TT::mfma(a.v, pb[kk], o_acc[dt]);
        }
      }
    }

    // ---- epilogue ----
    const float d_tot = d_part + __shfl_xor(d_part, 32, 64);
    const float inv = __builtin_amdgcn_rcpf(d_tot);
    if (row_ok) {
      T* dst = op + q_tok * p.o_sn + static_cast<int64_t>(head) * p.o_sh;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          x4 out;
#pragma unroll
          for (int j = 0; j < 4; ++j) out[j] = static_cast<T>(o_acc[dt][i4 * 4 + j] * inv);
          *reinterpret_cast<x4*>(dst + dt * 32 + i4 * 8 + g * 4) = out;
        }
      if (p.lse && g == 0)
        p.lse[q_tok * p.num_heads + head] = __builtin_amdgcn_logf(d_tot) + m_run * c;
    }
  }
}

template <typename T>
int launch(const FaParams& p, int64_t max_rows, hipStream_t stream) {
  static bool attr_set = false;
  if (!attr_set) {
    FO_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(&sparse_fa_kernel<T>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kSmemBytes));
    attr_set = true;
  }
  int num_cu = fo_num_cu();
  if (num_cu <= 0) return fo::fail(FO_ERR_HIP, "sparse_fa: no device");
  int64_t grid = 2 * static_cast<int64_t>(num_cu);
  if (grid > max_rows) grid = max_rows;
  sparse_fa_kernel<T><<<static_cast<unsigned>(grid), kThreads, kSmemBytes, stream>>>(p);
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
                                const int32_t* kv_blk_base, const int32_t* row_req,
                                const int32_t* row_qb, const int32_t* row_head,
                                const int32_t* kv_row_ptr, const int32_t* kv_idx, int32_t* counts,
                                int64_t max_rows, int32_t num_heads, int32_t head_dim,
                                int32_t block_q, int32_t block_kv, float sm_scale, void* stream) {
  FO_REQUIRE(head_dim == kHeadDim, "sparse_fa: head_dim %d is not supported (only 128)", head_dim);
  FO_REQUIRE(block_q == kBlockQ && block_kv == kBlockKV,
             "sparse_fa: sparse block sizes (%d, %d) are not supported (only 128, 128)", block_q,
             block_kv);
  FO_REQUIRE(dtype == FO_BF16 || dtype == FO_F16 || dtype == FO_FP8_E4M3,
             "sparse_fa: unsupported dtype code %d", dtype);
  FO_REQUIRE(num_heads > 0 && max_rows >= 0, "sparse_fa: bad sizes");
  if (max_rows == 0) return FO_OK;
  FO_REQUIRE(q && k && v && o && qo_indptr && kv_indptr && row_req && row_qb && row_head &&
                 kv_row_ptr && kv_idx && counts,
             "sparse_fa: null pointer");
  const int64_t strides[8] = {q_stride_n, q_stride_h, k_stride_n, k_stride_h,
                              v_stride_n, v_stride_h, o_stride_n, o_stride_h};
  for (int i = 0; i < 8; ++i)
    FO_REQUIRE(strides[i] % 8 == 0 && strides[i] > 0,
               "sparse_fa: strides must be positive multiples of 8 elements (128-bit accesses)");
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
  p.kv_row_ptr = kv_row_ptr; p.kv_idx = kv_idx; p.counts = counts;
  p.num_heads = num_heads; p.n_q_blocks = 0; p.n_kv_blocks = 0;
  p.sm_scale_log2 = sm_scale * 1.44269504088896340736f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == FO_BF16) return launch<__bf16>(p, max_rows, s);
  if (dtype == FO_F16) return launch<_Float16>(p, max_rows, s);
  return fo::fail(FO_ERR_INVALID, "sparse_fa: the fp8 path is not built yet");
}
