// fp8 e4m3fn block quantiser for gfx950: one absmax scale per (head, 128-token block).
// One workgroup per (block, head): the 128 x 128 slab is read once into registers (128-bit loads),
// reduced to its absmax (wave shuffles + LDS), then divided by scale = absmax/448 and converted with
// the hardware round-to-nearest-even e4m3 conversion; 2 bytes read + 1 byte written per element.
// Optionally a second e4m3 tensor takes the residual, x/scale - x8 rounded again, so that x8 + x8_lo
// carries x/scale to about 7 significant bits (a two-term operand for the fp8 matrix cores).
// The reference has no such kernel (its quantization.cuh only packs bits).
#include "fo_common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

constexpr int kThreads = 256;
constexpr int kBlock = 128;
constexpr float kFp8Max = 448.0f;

template <typename X8>
__global__ void __launch_bounds__(kThreads) quant_fp8_kernel(
    const void* __restrict__ xv, int64_t sn, int64_t sh, uint8_t* __restrict__ x8,
    uint8_t* __restrict__ x8_lo, float* __restrict__ scale, const int32_t* __restrict__ blk_tok0,
    const int32_t* __restrict__ blk_len, int32_t n_blk, int32_t num_heads) {
  using T = decltype(X8{}[0]);
  __shared__ float s_red[kThreads / 64];
  const int blk = blockIdx.x, head = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int tok0 = blk_tok0[blk], len = blk_len[blk];
  const int row0 = tid >> 4, col = (tid & 15) * 8;
  const char* x = static_cast<const char*>(xv);

  X8 v[8];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = row0 + 16 * i;
    if (r < len) {
      const int64_t off = (static_cast<int64_t>(tok0 + r) * sn + static_cast<int64_t>(head) * sh + col);
      v[i] = *reinterpret_cast<const X8*>(x + off * sizeof(T));
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(static_cast<float>(v[i][j])));
    }
  }
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
  if (lane == 0) s_red[wv] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
  const float s = amax > 0.f ? amax / kFp8Max : 1.0f;
  if (tid == 0) scale[static_cast<int64_t>(head) * n_blk + blk] = s;

#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = row0 + 16 * i;
    if (r < len) {
      float f[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        f[j] = static_cast<float>(v[i][j]) / s;
        f[j] = fminf(fmaxf(f[j], -kFp8Max), kFp8Max);
      }
      u32x2 out;
      unsigned w0 = 0, w1 = 0;
      w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], w0, false);
      w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w0, true);
      w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], w1, false);
      w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], w1, true);
      out[0] = w0;
      out[1] = w1;
      const int64_t o = (static_cast<int64_t>(tok0 + r) * num_heads + head) * kBlock + col;
      *reinterpret_cast<u32x2*>(x8 + o) = out;
      if (x8_lo) {
        typedef __attribute__((ext_vector_type(2))) float f32x2;
        const f32x2 h0 = __builtin_amdgcn_cvt_pk_f32_fp8(w0, false), h1 = __builtin_amdgcn_cvt_pk_f32_fp8(w0, true);
        const f32x2 h2 = __builtin_amdgcn_cvt_pk_f32_fp8(w1, false), h3 = __builtin_amdgcn_cvt_pk_f32_fp8(w1, true);
        unsigned l0 = 0, l1 = 0;
        l0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0] - h0[0], f[1] - h0[1], l0, false);
        l0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2] - h1[0], f[3] - h1[1], l0, true);
        l1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[4] - h2[0], f[5] - h2[1], l1, false);
        l1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[6] - h3[0], f[7] - h3[1], l1, true);
        u32x2 lo;
        lo[0] = l0;
        lo[1] = l1;
        *reinterpret_cast<u32x2*>(x8_lo + o) = lo;
      }
    }
  }
}

}  // namespace

extern "C" int fo_quant_fp8_block(const void* x, int dtype, int64_t x_stride_n, int64_t x_stride_h,
                                  uint8_t* x8, uint8_t* x8_lo, float* scale, const int32_t* blk_tok0,
                                  const int32_t* blk_len, int32_t n_blk, int32_t num_heads,
                                  int32_t head_dim, void* stream) {
  FO_REQUIRE(dtype == FO_BF16 || dtype == FO_F16, "quant_fp8: input must be bf16 or fp16");
  FO_REQUIRE(head_dim == kBlock, "quant_fp8: head_dim %d is not supported (only 128)", head_dim);
  FO_REQUIRE(n_blk >= 0 && num_heads > 0 && num_heads <= 65535, "quant_fp8: bad sizes");
  if (n_blk == 0) return FO_OK;
  FO_REQUIRE(x && x8 && scale && blk_tok0 && blk_len, "quant_fp8: null pointer");
  FO_REQUIRE(x_stride_n % 8 == 0 && x_stride_h % 8 == 0 &&
                 (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(x8) & 7) == 0 &&
                 (reinterpret_cast<uintptr_t>(x8_lo) & 7) == 0,
             "quant_fp8: x must be 16-byte aligned with strides that are multiples of 8");
  dim3 grid(n_blk, num_heads);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == FO_BF16) {
    quant_fp8_kernel<bf16x8><<<grid, kThreads, 0, s>>>(x, x_stride_n, x_stride_h, x8, x8_lo, scale,
                                                      blk_tok0, blk_len, n_blk, num_heads);
  } else {
    quant_fp8_kernel<f16x8><<<grid, kThreads, 0, s>>>(x, x_stride_n, x_stride_h, x8, x8_lo, scale,
                                                     blk_tok0, blk_len, n_blk, num_heads);
  }
  FO_CHECK_LAUNCH();
  return FO_OK;
}
