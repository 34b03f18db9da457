// fp8 e4m3fn block quantiser for gfx950: one absmax scale per (head, 128-token block).
// One workgroup per (block, head): the 128 x 128 slab is read once into registers (128-bit loads),
// reduced to its absmax (wave shuffles + LDS), then divided by scale = absmax/448 and converted with
// the hardware round-to-nearest-even e4m3 conversion (128-bit stores); 2 bytes read + 1 byte written
// per element.
// Optionally a second e4m3 tensor takes the residual, x/scale - x8 rounded again, so that x8 + x8_lo
// carries x/scale to about 7 significant bits (a two-term operand for the fp8 matrix cores).
// The reference has no such kernel (its quantization.cuh only packs bits).
#include "fo_common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;

constexpr int kThreads = 256;
constexpr int kBlock = 128;
constexpr float kFp8Max = 448.0f;
constexpr int kChunks = 4;  // 16-element pieces of a slab per thread

// The slab's elements all divide by the same scale s, and an IEEE division costs about a dozen vector
// instructions: at 64 of them per thread the kernel was bound by the vector ALU, not by memory.  With
// y = 1 / s rounded correctly, q0 = x * y, e = s * q0 - x (one fused operation, exact) and
// q = q0 - e * y (fused), q is the correctly rounded x / s: checked on the device against the
// division instruction sequence for all 2^16 bf16 and all 2^16 fp16 values of x under every positive
// finite 16-bit absmax with s >= 2^-80 (2 * 10^9 pairs): identical fp32 bits wherever
// |x / s| > 2^-33, identical e4m3 bytes (and residual bytes) everywhere, signed zeros included (the
// order of the operands above is what keeps -0).  Slabs outside that range (an infinite or NaN
// absmax, s < 2^-80) take the division.
template <bool kFast>
__device__ __forceinline__ float quotient(float x, float s, float y) {
  if (!kFast) return x / s;
  const float q0 = x * y;
  const float e = __builtin_fmaf(s, q0, -x);
  return __builtin_fmaf(-e, y, q0);
}

template <typename X8, bool kFast>
__device__ __forceinline__ void quantise_chunks(const X8 (&v)[2 * kChunks], float s, int row0, int col, int len,
                                                int64_t out0, int64_t out_row, uint8_t* __restrict__ x8,
                                                uint8_t* __restrict__ x8_lo) {
  const float y = 1.0f / s;
#pragma unroll
  for (int i = 0; i < kChunks; ++i) {
    const int r = row0 + (kBlock / kChunks) * i;
    if (r >= len) continue;
    float f[16];
#pragma unroll
    for (int j = 0; j < 16; ++j)
      f[j] = __builtin_amdgcn_fmed3f(quotient<kFast>(static_cast<float>(v[2 * i + (j >> 3)][j & 7]), s, y),
                                     -kFp8Max, kFp8Max);
    u32x4 w;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      unsigned t = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j], f[4 * j + 1], 0u, false);
      w[j] = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j + 2], f[4 * j + 3], t, true);
    }
    const int64_t o = out0 + static_cast<int64_t>(r) * out_row + col;
    // (streaming stores: the bytes are not read again by this kernel; +1.5 % at the Wan size)
    __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(x8 + o));
    if (x8_lo) {
      u32x4 lo;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x2 h0 = __builtin_amdgcn_cvt_pk_f32_fp8(w[j], false), h1 = __builtin_amdgcn_cvt_pk_f32_fp8(w[j], true);
        unsigned t = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j] - h0[0], f[4 * j + 1] - h0[1], 0u, false);
        lo[j] = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j + 2] - h1[0], f[4 * j + 3] - h1[1], t, true);
      }
      __builtin_nontemporal_store(lo, reinterpret_cast<u32x4*>(x8_lo + o));
    }
  }
}

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
  // a thread takes 16 consecutive elements of a row (two 16-byte loads, one 16-byte store per
  // output), eight threads a row, the workgroup 32 rows at a time
  const int row0 = tid >> 3, col = (tid & 7) * 16;
  const char* x = static_cast<const char*>(xv);

  X8 v[2 * kChunks];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < kChunks; ++i) {
    const int r = row0 + (kBlock / kChunks) * i;
    if (r < len) {
      const int64_t off = (static_cast<int64_t>(tok0 + r) * sn + static_cast<int64_t>(head) * sh + col);
      v[2 * i] = *reinterpret_cast<const X8*>(x + off * sizeof(T));
      v[2 * i + 1] = *reinterpret_cast<const X8*>(x + (off + 8) * sizeof(T));
    }
  }
#pragma unroll
  for (int i = 0; i < kChunks; ++i) {
    if (row0 + (kBlock / kChunks) * i < len) {
#pragma unroll
      for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fabsf(static_cast<float>(v[2 * i + (j >> 3)][j & 7])));
    }
  }
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
  if (lane == 0) s_red[wv] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
  const float s = amax > 0.f ? amax / kFp8Max : 1.0f;
  if (tid == 0) scale[static_cast<int64_t>(head) * n_blk + blk] = s;
  const int64_t out0 = (static_cast<int64_t>(tok0) * num_heads + head) * kBlock;
  const int64_t out_row = static_cast<int64_t>(num_heads) * kBlock;
  if (amax < __builtin_inff() && s >= 0x1p-80f) {  // (uniform over the workgroup)
    quantise_chunks<X8, true>(v, s, row0, col, len, out0, out_row, x8, x8_lo);
  } else {
    quantise_chunks<X8, false>(v, s, row0, col, len, out0, out_row, x8, x8_lo);
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
                 (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(x8) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(x8_lo) & 15) == 0,
             "quant_fp8: x, x8 and x8_lo must be 16-byte aligned, the strides of x multiples of 8");
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
