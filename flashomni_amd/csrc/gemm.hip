// GEMM-Q and GEMM-O (with reduction) for gfx950: MFMA tile GEMMs that skip work according to the
// bit-packed (token-block, head) flags.
//
//   GEMM-Q  y[b, iy-tile, ix-tile] = x[b, iy-tile, :] . w[ix-tile, :]^T + bias   for flagged tiles;
//           the other tiles are never touched (reference: gemm/w16a16/gemm.cuh:50-58, 83-92).
//   GEMM-O  y[b, iy-tile, :] = init + sum_{selected heads h} x[:, h-slice] . w[:, h-slice]^T
//           where unselected head slices are never loaded
//           (reference: gemm/w16a16/gemm_reduction.cuh:77-95, 126-160).
//
// One workgroup = 256 lanes = 2x2 wavefronts on a 128x128 output tile, BK = 64, two LDS stages fed
// through registers with 128-bit accesses, one barrier per k step.  The product is formed
// transposed (A operand = W rows, B operand = X rows) so that in the 32x32 accumulator layout a
// lane owns one output row and runs of 4 consecutive columns: the epilogue then reads the init
// matrix and writes the result with 8/16-byte accesses without going through LDS.
// fp32 accumulation starts from the init value converted to fp32; one round-to-nearest cast at
// the end.
#include "fo_common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

constexpr int kThreads = 256;
constexpr int kTile = 128;  // output tile edge; also the granularity of the skip flags
constexpr int kBK = 64;
constexpr int kRowStride = 144;  // bytes per LDS row: 64 elements + 16 B pad
constexpr int kOperandBytes = kTile * kRowStride;
constexpr int kStageBytes = 2 * kOperandBytes;
constexpr int kSmemBytes = 2 * kStageBytes;
constexpr int kMaxHeads = 256;

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
  int32_t m, n, k;
  int32_t sparse_q_size, num_heads, head_dim, num_text_tokens;
  int32_t flag;       // GEMM-Q: is_full.  GEMM-O: is_for_cached
  int32_t bias_kind;  // FO_BIAS_*
  int32_t bias_f32;   // matrix bias is fp32
  int32_t y_f32;      // output is fp32
};

// kReduce = false: GEMM-Q.  kReduce = true: GEMM-O.
template <typename T, bool kReduce>
__global__ void __launch_bounds__(kThreads, 2) gemm_kernel(const GemmParams p) {
  using TT = Types<T>;
  using x8 = typename TT::x8;
  using x4 = typename TT::x4;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  __shared__ int32_t s_heads[kMaxHeads];
  __shared__ int32_t s_nsel;

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int wm = wv >> 1, wn = wv & 1;
  const int ix = blockIdx.x, iy = blockIdx.y, bz = blockIdx.z;

  const uint8_t* info = p.sparse_info ? p.sparse_info + p.sparse_info_indptr[bz] : nullptr;
  const uint32_t flag_base =
      static_cast<uint32_t>(p.num_text_tokens + iy * kTile) / p.sparse_q_size * p.num_heads;

  int n_iter;
  if constexpr (!kReduce) {
    if (!p.flag) {
      const uint32_t bit = flag_base + static_cast<uint32_t>(ix * kTile) / p.head_dim;
      if (!((info[bit >> 3] >> (bit & 7)) & 1)) return;
    }
    n_iter = (p.k + kBK - 1) / kBK;
  } else {
    // selected head slices of this row tile, ascending
    if (wv == 0) {
      int count = 0;
      const int n_slices = p.k / p.head_dim;
      for (int h0 = 0; h0 < n_slices; h0 += 64) {
        const int h = h0 + lane;
        bool sel = false;
        if (h < n_slices) {
          const uint32_t bit = flag_base + h;
          const bool one = (info[bit >> 3] >> (bit & 7)) & 1;
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
  }
  const int iters_per_head = kReduce ? p.head_dim / kBK : 1;

  const T* __restrict__ xp = static_cast<const T*>(p.x) + static_cast<int64_t>(bz) * p.m * p.k;
  const T* __restrict__ wp = static_cast<const T*>(p.w);

  // staging: chunk cc = tid + 256*i -> tile row cc/8 (32 rows per pass), 16-byte column cc%8
  const int st_row = tid >> 3, st_col = tid & 7;
  u32x4 xst[4], wst[4];
  auto k_of = [&](int it) -> int {
    if constexpr (kReduce) {
      return s_heads[it / iters_per_head] * p.head_dim + (it % iters_per_head) * kBK;
    } else {
      return it * kBK;
    }
  };
  auto load_tiles = [&](int it) {
    const int k0 = k_of(it) + st_col * 8;
    const bool k_ok = k0 < p.k;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = st_row + 32 * i;
      int xm = iy * kTile + r;
      xm = xm < p.m ? xm : p.m - 1;
      const u32x4 z = {0u, 0u, 0u, 0u};
      xst[i] = k_ok ? *reinterpret_cast<const u32x4*>(xp + static_cast<int64_t>(xm) * p.k + k0) : z;
      wst[i] = k_ok ? *reinterpret_cast<const u32x4*>(
                          wp + static_cast<int64_t>(ix * kTile + r) * p.k + k0)
                    : z;
    }
  };

  // accumulators acc[nt][mt]: n = wn*64 + nt*32 + (i/4)*8 + g*4 + i%4, m = wm*64 + mt*32 + l32
  f32x16 acc[2][2];
  const int64_t y_batch = static_cast<int64_t>(bz) * p.m * p.n;
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
      const int mrow = iy * kTile + wm * 64 + mt * 32 + l32;
      const int mrow_c = mrow < p.m ? mrow : p.m - 1;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int ncol = ix * kTile + wn * 64 + nt * 32 + i4 * 8 + g * 4;
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

  if (n_iter > 0) load_tiles(0);
  for (int it = 0; it < n_iter; ++it) {
    uint8_t* xs = smem + (it & 1) * kStageBytes;
    uint8_t* ws = xs + kOperandBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = st_row + 32 * i;
      *reinterpret_cast<u32x4*>(xs + r * kRowStride + st_col * 16) = xst[i];
      *reinterpret_cast<u32x4*>(ws + r * kRowStride + st_col * 16) = wst[i];
    }
    __syncthreads();
    if (it + 1 < n_iter) load_tiles(it + 1);
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      x8 a[2], b[2];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
        a[nt] = *reinterpret_cast<const x8*>(ws + (wn * 64 + nt * 32 + l32) * kRowStride + ks * 32 +
                                             g * 16);
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
        b[mt] = *reinterpret_cast<const x8*>(xs + (wm * 64 + mt * 32 + l32) * kRowStride + ks * 32 +
                                             g * 16);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) acc[nt][mt] = TT::mfma(a[nt], b[mt], acc[nt][mt]);
    }
  }

  // epilogue
#pragma unroll
  for (int mt = 0; mt < 2; ++mt) {
    const int mrow = iy * kTile + wm * 64 + mt * 32 + l32;
    if (mrow >= p.m) continue;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int ncol = ix * kTile + wn * 64 + nt * 32 + i4 * 8 + g * 4;
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

template <typename T, bool kReduce>
int launch(const GemmParams& p, int batch, hipStream_t stream) {
  static bool attr_set = false;
  if (!attr_set) {
    FO_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<T, kReduce>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kSmemBytes));
    attr_set = true;
  }
  dim3 grid(p.n / kTile, (p.m + kTile - 1) / kTile, batch);
  gemm_kernel<T, kReduce><<<grid, kThreads, kSmemBytes, stream>>>(p);
  FO_CHECK_LAUNCH();
  return FO_OK;
}

int check_common(const void* x, const void* w, void* y, int dtype, int32_t batch, int32_t m,
                 int32_t n, int32_t k, int32_t sparse_q_size, int32_t num_qo_heads) {
  FO_REQUIRE(dtype == FO_BF16 || dtype == FO_F16, "gemm: only bf16 / fp16 operands are supported");
  FO_REQUIRE(batch > 0 && m > 0 && n > 0 && k > 0, "gemm: bad shape");
  FO_REQUIRE(n % 128 == 0 && k % 32 == 0, "only support N %% 128 == 0, K %% 32 == 0 (got N=%d K=%d)",
             n, k);
  FO_REQUIRE(batch <= 65535 && (m + kTile - 1) / kTile <= 65535, "gemm: grid too large");
  FO_REQUIRE(sparse_q_size > 0 && num_qo_heads > 0 && n % num_qo_heads == 0,
             "gemm: bad sparse_q_size / num_qo_heads");
  FO_REQUIRE(x && w && y, "gemm: null pointer");
  FO_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) |
               reinterpret_cast<uintptr_t>(y)) & 15) == 0,
             "gemm: x, w, y must be 16-byte aligned");
  return FO_OK;
}

}  // namespace

extern "C" int fo_gemm_q(const void* x, const void* w, const void* bias, void* y, int dtype,
                         int32_t batch, int32_t m, int32_t n, int32_t k, int32_t sparse_q_size,
                         int32_t num_qo_heads, const uint8_t* sparse_info,
                         const int32_t* sparse_info_indptr, int32_t num_text_tokens, int is_full,
                         void* stream) {
  if (int rc = check_common(x, w, y, dtype, batch, m, n, k, sparse_q_size, num_qo_heads)) return rc;
  FO_REQUIRE(is_full || (sparse_info && sparse_info_indptr),
             "gemm: sparse_info and sparse_info_indptr are required unless is_full");
  FO_REQUIRE(num_text_tokens >= 0, "gemm: negative num_text_tokens");
  FO_REQUIRE(!bias || (reinterpret_cast<uintptr_t>(bias) & 7) == 0, "gemm: bias must be 8-byte aligned");
  GemmParams p{};
  p.x = x; p.w = w; p.bias = bias; p.y = y;
  p.sparse_info = is_full ? nullptr : sparse_info;
  p.sparse_info_indptr = sparse_info_indptr;
  p.m = m; p.n = n; p.k = k;
  p.sparse_q_size = sparse_q_size; p.num_heads = num_qo_heads; p.head_dim = n / num_qo_heads;
  p.num_text_tokens = num_text_tokens;
  p.flag = is_full ? 1 : 0;
  p.bias_kind = bias ? FO_BIAS_VECTOR : FO_BIAS_NONE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dtype == FO_BF16 ? launch<__bf16, false>(p, batch, s) : launch<_Float16, false>(p, batch, s);
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
  p.m = m; p.n = n; p.k = k;
  p.sparse_q_size = sparse_q_size; p.num_heads = num_qo_heads; p.head_dim = head_dim;
  p.num_text_tokens = num_text_tokens;
  p.flag = is_for_cached ? 1 : 0;
  p.bias_kind = bias_kind;
  p.bias_f32 = bias_dtype == FO_F32;
  p.y_f32 = y_dtype == FO_F32;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dtype == FO_BF16 ? launch<__bf16, true>(p, batch, s) : launch<_Float16, true>(p, batch, s);
}
