// packbits / segment_packbits for gfx950: eight bool bytes are gathered into one output byte with a
// multiply (aligned packbits: 64 bools per lane, four 16-byte loads and one 8-byte store);
// HBM-bound (n bytes read, n/8 written).
// Semantics: numpy.packbits per segment (reference: include/flashomni/quantization.cuh:39-83).
#include "fo_common.h"

namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ uint8_t pack8(uint64_t bools, int little) {
  // normalise every byte to 0/1
  uint64_t nz = bools | (bools >> 4);
  nz |= nz >> 2;
  nz |= nz >> 1;
  nz &= 0x0101010101010101ull;
  // byte j (memory order) carries element j.  little: bit j.  big: bit 7-j.
  const uint64_t mul = little ? 0x0102040810204080ull : 0x8040201008040201ull;
  return static_cast<uint8_t>((nz * mul) >> 56);
}

__device__ __forceinline__ uint64_t load8_guarded(const uint8_t* p, int64_t remaining) {
  // `remaining` bytes are readable at p; missing ones read as 0
  if (remaining >= 8 && (reinterpret_cast<uintptr_t>(p) & 7) == 0) {
    return *reinterpret_cast<const uint64_t*>(p);
  }
  uint64_t v = 0;
  const int n = remaining < 8 ? static_cast<int>(remaining) : 8;
  for (int j = 0; j < n; ++j) v |= static_cast<uint64_t>(p[j]) << (8 * j);
  return v;
}

// kVec: x is 16-byte and y 8-byte aligned: a lane turns 64 bools (four 16-byte loads, all in flight
// together) into one 8-byte store; the last n % 64 bools go the byte-wise way.
template <bool kVec>
__global__ void __launch_bounds__(kThreads) packbits_kernel(const uint8_t* __restrict__ x,
                                                            int64_t n, int little,
                                                            uint8_t* __restrict__ y) {
  typedef __attribute__((ext_vector_type(2))) uint64_t u64x2;
  const int64_t nbytes = (n + 7) >> 3;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  int64_t done = 0;  // output bytes covered by the vector part
  if constexpr (kVec) {
    const int64_t nvec = n >> 6;
    for (int64_t v = tid; v < nvec; v += stride) {
      const u64x2* src = reinterpret_cast<const u64x2*>(x + v * 64);
      const u64x2 a = src[0], b = src[1], c = src[2], d = src[3];
      const uint64_t out = static_cast<uint64_t>(pack8(a[0], little)) | static_cast<uint64_t>(pack8(a[1], little)) << 8 |
                           static_cast<uint64_t>(pack8(b[0], little)) << 16 | static_cast<uint64_t>(pack8(b[1], little)) << 24 |
                           static_cast<uint64_t>(pack8(c[0], little)) << 32 | static_cast<uint64_t>(pack8(c[1], little)) << 40 |
                           static_cast<uint64_t>(pack8(d[0], little)) << 48 | static_cast<uint64_t>(pack8(d[1], little)) << 56;
      *reinterpret_cast<uint64_t*>(y + v * 8) = out;
    }
    done = nvec * 8;
  }
  for (int64_t i = done + tid; i < nbytes; i += stride) {
    y[i] = pack8(load8_guarded(x + i * 8, n - i * 8), little);
  }
}

__global__ void __launch_bounds__(kThreads) segment_packbits_kernel(
    const uint8_t* __restrict__ x, const int32_t* __restrict__ in_indptr,
    const int32_t* __restrict__ out_indptr, int little, uint8_t* __restrict__ y) {
  const int seg = blockIdx.y;
  const int64_t begin = in_indptr[seg];
  const int64_t n = in_indptr[seg + 1] - begin;
  const int64_t nbytes = (n + 7) >> 3;
  const int64_t out0 = out_indptr[seg];
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < nbytes;
       i += stride) {
    y[out0 + i] = pack8(load8_guarded(x + begin + i * 8, n - i * 8), little);
  }
}

int grid_for(int64_t nbytes) {
  int64_t g = (nbytes + kThreads - 1) / kThreads;
  if (g < 1) g = 1;
  if (g > 256 * 16) g = 256 * 16;
  return static_cast<int>(g);
}

}  // namespace

extern "C" int fo_packbits(const uint8_t* x, int64_t n, int bitorder, uint8_t* y, void* stream) {
  FO_REQUIRE(bitorder == FO_BITORDER_BIG || bitorder == FO_BITORDER_LITTLE,
             "bitorder must be 'big' or 'little'");
  FO_REQUIRE(n >= 0, "packbits: negative length");
  if (n == 0) return FO_OK;
  FO_REQUIRE(x && y, "packbits: null pointer");
  const bool vec = n >= 64 && ((reinterpret_cast<uintptr_t>(x) & 15) | (reinterpret_cast<uintptr_t>(y) & 7)) == 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (vec) {
    packbits_kernel<true><<<grid_for((n + 63) / 64), kThreads, 0, s>>>(x, n, bitorder == FO_BITORDER_LITTLE, y);
  } else {
    packbits_kernel<false><<<grid_for((n + 7) / 8), kThreads, 0, s>>>(x, n, bitorder == FO_BITORDER_LITTLE, y);
  }
  FO_CHECK_LAUNCH();
  return FO_OK;
}

extern "C" int fo_segment_packbits(const uint8_t* x, const int32_t* in_indptr,
                                   const int32_t* out_indptr, int32_t num_segments, int bitorder,
                                   uint8_t* y, void* stream) {
  FO_REQUIRE(bitorder == FO_BITORDER_BIG || bitorder == FO_BITORDER_LITTLE,
             "bitorder must be 'big' or 'little'");
  FO_REQUIRE(num_segments >= 0 && num_segments <= 65535, "segment_packbits: bad segment count %d",
             num_segments);
  if (num_segments == 0) return FO_OK;
  FO_REQUIRE(in_indptr && out_indptr, "segment_packbits: null indptr");
  // segment lengths live on the device: use a fixed, generous x-grid and stride inside
  dim3 grid(num_segments == 1 ? 1024 : 64, num_segments);
  segment_packbits_kernel<<<grid, kThreads, 0, static_cast<hipStream_t>(stream)>>>(
      x, in_indptr, out_indptr, bitorder == FO_BITORDER_LITTLE, y);
  FO_CHECK_LAUNCH();
  return FO_OK;
}
