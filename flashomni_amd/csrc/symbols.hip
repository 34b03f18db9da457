// Symbol producer for gfx950: pooled attention scores -> bit-packed sparse_info / sparse_kv_info
// in the layout the decoder and the GEMMs read (bit = q_block * H + head, resp.
// (q_block * H + head) * NKV + kv_block; little-endian bytes; one byte-aligned segment per request).
//
// Procedure (reference: benchmark/test_attn_score.py:93-128 with the fill kernels of :5-91): a row
// of scores is soft-maxed, and the entries of lowest score whose cumulative probability stays within
// a threshold get symbol 0.  The reference sorts, takes a cumulative sum and searches it; here one
// wavefront owns a row in registers and finds the cut directly: probabilities become 2^-30
// fixed-point integers (integer sums do not depend on the order of addition, so the result is the
// same whichever lanes hold which entries), scores become order-preserving 32-bit keys, and 32
// steps of bisection over the key space find the largest key bound whose mass below fits.  Equal
// scores at the cut are taken in index order, as a stable sort would.
//
// One launch, one pass over the scores (4 B per entry read, 1/8 B written); eight consecutive rows
// of a request make one workgroup, so every workgroup owns whole output bytes and nothing needs
// atomics or a cleared output.
#include "fo_common.h"

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kRowsPerGroup = 8;
constexpr int kMaxBlocks = 4096;
constexpr float kFixedOne = 1073741824.0f;  // 2^30

template <typename T>
__device__ __forceinline__ float to_f32(T v);
template <>
__device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ float to_f32<__hip_bfloat16>(__hip_bfloat16 v) {
  return __bfloat162float(v);
}
template <>
__device__ __forceinline__ float to_f32<__half>(__half v) { return __half2float(v); }

// ascending float order -> ascending unsigned order; 0xffffffff is kept free for padding
__device__ __forceinline__ uint32_t order_key(float s) {
  const uint32_t u = __float_as_uint(s);
  const uint32_t k = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  return k < 0xfffffffeu ? k : 0xfffffffeu;
}

// sum over the 64 lanes, returned in every lane (uniform: built from scalar reads of four lanes)
__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
  v += __builtin_amdgcn_update_dpp(0u, v, 0xb1, 0xf, 0xf, true);   // quad_perm [1,0,3,2]
  v += __builtin_amdgcn_update_dpp(0u, v, 0x4e, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
  v += __builtin_amdgcn_update_dpp(0u, v, 0x141, 0xf, 0xf, true);  // row_half_mirror
  v += __builtin_amdgcn_update_dpp(0u, v, 0x140, 0xf, 0xf, true);  // row_mirror
  return __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) +
         __builtin_amdgcn_readlane(v, 32) + __builtin_amdgcn_readlane(v, 48);
}

__device__ __forceinline__ float wave_max_f32(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const uint32_t o = static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), off));
    v = o > v ? o : v;
  }
  return v;
}

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

// One row held by one wavefront: entry i sits in lane i % 64, slot i / 64.  On return drop[e] says
// whether entry (e * 64 + lane) gets symbol 0.  `threshold` is the admitted cumulative probability.
template <int E>
__device__ __forceinline__ void select_low_mass(const float (&score)[E], int n, float threshold,
                                                int lane, bool (&drop)[E]) {
  uint32_t key[E], w[E];
  float m = -INFINITY;
#pragma unroll
  for (int e = 0; e < E; ++e)
    if (e * 64 + lane < n) m = fmaxf(m, score[e]);
  m = wave_max_f32(m);
  float ex[E], z = 0.f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const bool valid = e * 64 + lane < n;
    ex[e] = valid ? __expf(score[e] - m) : 0.f;
    z += ex[e];
    key[e] = valid ? order_key(score[e]) : 0xffffffffu;
  }
  z = wave_sum_f32(z);
  const float scale = kFixedOne / z;
#pragma unroll
  for (int e = 0; e < E; ++e) w[e] = static_cast<uint32_t>(ex[e] * scale + 0.5f);
  const float t = fminf(fmaxf(threshold, 0.f), 1.5f);
  const uint32_t budget = static_cast<uint32_t>(t * kFixedOne);

  // largest bound x with  sum{ w : key < x } <= budget
  uint32_t x = 0, below = 0;
  for (int bit = 31; bit >= 0; --bit) {
    const uint32_t c = x | (1u << bit);
    uint32_t part = 0;
#pragma unroll
    for (int e = 0; e < E; ++e) part += key[e] < c ? w[e] : 0u;
    const uint32_t g = wave_sum_u32(part);
    if (g <= budget) {
      x = c;
      below = g;
    }
  }
  // entries whose key equals x straddle the cut: admit them in index order while they fit
  uint32_t tie_w = 0;
#pragma unroll
  for (int e = 0; e < E; ++e)
    if (key[e] == x && w[e] > tie_w) tie_w = w[e];
  tie_w = __builtin_amdgcn_readfirstlane(wave_max_u32(tie_w));
  const uint32_t room = budget - below;
  const uint32_t extra = tie_w ? room / tie_w : 0xffffffffu;
  uint32_t seen = 0;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const bool tie = key[e] == x && x != 0xffffffffu;
    const uint64_t mask = __ballot(tie);
    const uint32_t rank = seen + __popcll(mask & ((1ull << lane) - 1ull));
    drop[e] = key[e] < x || (tie && rank < extra);
    seen += __popcll(mask);
  }
}

struct ProducerArgs {
  const void* scores;           // [batch, H, NQ, NK]
  const float* q_threshold;     // [batch]
  const float* kv_threshold;    // [H]
  uint8_t* sparse_info;         // batch * ceil(NQ*H / 8) bytes
  uint8_t* sparse_kv_info;      // batch * ceil(NQ*H*NK / 8) bytes
  int32_t* sparse_info_indptr;     // [batch + 1] byte offsets (written)
  int32_t* sparse_kv_info_indptr;  // [batch + 1] byte offsets (written)
  int32_t batch, heads, n_q, n_k, text_q, text_kv;
};

__device__ __forceinline__ uint8_t gather8(uint64_t flags) {
  // eight 0/1 bytes -> one byte, entry j in bit j
  return static_cast<uint8_t>((flags * 0x0102040810204080ull) >> 56);
}

// ---- q symbols: one workgroup per request --------------------------------------------------------
// The H * n_text_q contributing rows are split into `parts` interleaved subsets; a wavefront sums
// one subset over one 64-column chunk (coalesced 256 B loads, eight in flight), and the partial sums
// are added in subset order, so the result does not depend on which wavefront did what.
// LDS (carved from the launch's dynamic block): partial sums [parts][width], sums [width], keep
// flags [n_q + 8].
struct QJobLayout {
  int width, parts;
  size_t bytes;
};

__host__ __device__ inline QJobLayout q_job_layout(int n_q, int n_k, int text_kv) {
  QJobLayout l;
  l.width = ((n_k - text_kv + 63) / 64) * 64;
  if (l.width < 64) l.width = 64;
  int parts = (16384 - n_q - 16) / (4 * l.width) - 1;
  l.parts = parts < 1 ? 1 : (parts > 16 ? 16 : parts);
  l.bytes = static_cast<size_t>(4) * l.width * (l.parts + 1) + n_q + 16;
  return l;
}

template <typename T, int E>
__device__ __forceinline__ void q_symbols_job(const ProducerArgs& a, int b, uint8_t* lds) {
  const QJobLayout lay = q_job_layout(a.n_q, a.n_k, a.text_kv);
  const int width = lay.width, parts = lay.parts;
  float* s_part = reinterpret_cast<float*>(lds);
  float* s_sum = s_part + parts * width;
  uint8_t* s_keep = reinterpret_cast<uint8_t*>(s_sum + width);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n_img = a.n_k - a.text_kv;
  const int chunks = (n_img + 63) >> 6;
  const int n_rows = a.heads * a.text_q;
  const T* base = static_cast<const T*>(a.scores) + static_cast<int64_t>(b) * a.heads * a.n_q * a.n_k;
  constexpr int kFlight = 8;
  for (int item = wave; item < chunks * parts; item += kWaves) {
    const int c = item / parts, part = item - c * parts;
    const int j = c * 64 + lane;
    float acc[kFlight];
#pragma unroll
    for (int u = 0; u < kFlight; ++u) acc[u] = 0.f;
    if (j < n_img) {
      const T* col = base + a.text_kv + j;
      int r = part;
      for (; r + (kFlight - 1) * parts < n_rows; r += kFlight * parts) {
#pragma unroll
        for (int u = 0; u < kFlight; ++u) {
          const int row = r + u * parts;             // row = head * n_text_q + q
          const int h = row / a.text_q, q = row - h * a.text_q;
          acc[u] += to_f32(col[(static_cast<int64_t>(h) * a.n_q + q) * a.n_k]);
        }
      }
      for (; r < n_rows; r += parts) {
        const int h = r / a.text_q, q = r - h * a.text_q;
        acc[0] += to_f32(col[(static_cast<int64_t>(h) * a.n_q + q) * a.n_k]);
      }
    }
    float total = 0.f;
#pragma unroll
    for (int u = 0; u < kFlight; ++u) total += acc[u];
    s_part[part * width + j] = total;
  }
  for (int q = tid; q < a.n_q + 8; q += kThreads) s_keep[q] = q < a.n_q ? 1 : 0;
  __syncthreads();
  for (int j = tid; j < n_img; j += kThreads) {
    float acc = 0.f;
    for (int part = 0; part < parts; ++part) acc += s_part[part * width + j];
    s_sum[j] = acc;
  }
  __syncthreads();
  if (tid < 64 && n_img > 0) {
    float score[E];
    bool drop[E];
#pragma unroll
    for (int e = 0; e < E; ++e) score[e] = e * 64 + lane < n_img ? s_sum[e * 64 + lane] : 0.f;
    select_low_mass<E>(score, n_img, a.q_threshold[b], lane, drop);
#pragma unroll
    for (int e = 0; e < E; ++e)
      if (e * 64 + lane < n_img && drop[e]) s_keep[a.text_q + e * 64 + lane] = 0;
  }
  __syncthreads();
  const int bits = a.n_q * a.heads;
  const int nbytes = (bits + 7) >> 3;
  uint8_t* out = a.sparse_info + static_cast<int64_t>(b) * nbytes;
  for (int k = tid; k < nbytes; k += kThreads) {
    uint32_t byte = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int f = 8 * k + i;
      if (f < bits) byte |= static_cast<uint32_t>(s_keep[f / a.heads]) << i;
    }
    out[k] = static_cast<uint8_t>(byte);
  }
  if (tid == 0) {
    a.sparse_info_indptr[b + 1] = (b + 1) * nbytes;
    if (b == 0) a.sparse_info_indptr[0] = 0;
  }
}

// ---- one launch: workgroups [0, batch) make the q symbols of a request each (they start first and
// run beside the rest); every other workgroup makes the kv symbols of eight consecutive
// (q_block, head) rows of a request ------------------------------------------------------------------
template <typename T, int E>
__global__ void __launch_bounds__(kThreads) symbols_kernel(ProducerArgs a, int groups_per_request) {
  extern __shared__ __align__(16) uint8_t s_flags[];  // kv job: kRowsPerGroup * n_k (+8) keep flags
  if (static_cast<int>(blockIdx.x) < a.batch) {
    q_symbols_job<T, E>(a, blockIdx.x, s_flags);
    return;
  }
  const int block = blockIdx.x - a.batch;
  const int b = block / groups_per_request;
  const int g = block - b * groups_per_request;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rows = a.n_q * a.heads;
  const int row0 = g * kRowsPerGroup;
  const int rows_here = min(kRowsPerGroup, rows - row0);
  const T* base = static_cast<const T*>(a.scores) + static_cast<int64_t>(b) * a.heads * a.n_q * a.n_k;

  for (int r = wave; r < rows_here; r += kWaves) {
    const int row = row0 + r;
    const int qb = row / a.heads, h = row - qb * a.heads;
    uint8_t* flags = s_flags + r * a.n_k;
    if (qb < a.text_q) {
#pragma unroll
      for (int e = 0; e < E; ++e)
        if (e * 64 + lane < a.n_k) flags[e * 64 + lane] = 1;
      continue;
    }
    const T* src = base + (static_cast<int64_t>(h) * a.n_q + qb) * a.n_k;
    float score[E];
    bool drop[E];
#pragma unroll
    for (int e = 0; e < E; ++e) score[e] = e * 64 + lane < a.n_k ? to_f32(src[e * 64 + lane]) : 0.f;
    select_low_mass<E>(score, a.n_k, a.kv_threshold[h], lane, drop);
#pragma unroll
    for (int e = 0; e < E; ++e)
      if (e * 64 + lane < a.n_k) flags[e * 64 + lane] = drop[e] ? 0 : 1;
  }
  const int bits_here = rows_here * a.n_k;
  if (tid < 8) s_flags[bits_here + tid] = 0;  // padding bits of a request's last byte
  __syncthreads();

  const int64_t seg_bytes = (static_cast<int64_t>(rows) * a.n_k + 7) >> 3;
  uint8_t* out = a.sparse_kv_info + b * seg_bytes + static_cast<int64_t>(g) * a.n_k;  // 8 rows = n_k bytes
  const int nbytes = (bits_here + 7) >> 3;
  for (int k = tid; k < nbytes; k += kThreads)
    out[k] = gather8(*reinterpret_cast<const uint64_t*>(s_flags + 8 * k));
  if (g == 0 && tid == 0) {
    a.sparse_kv_info_indptr[b + 1] = static_cast<int32_t>((b + 1) * seg_bytes);
    if (b == 0) a.sparse_kv_info_indptr[0] = 0;
  }
}

constexpr int kSlots[] = {1, 2, 4, 6, 8, 10, 12, 16, 24, 32, 48, 64};

template <typename T, int E>
int launch_both(const ProducerArgs& a, hipStream_t stream) {
  // the q job holds n_k - n_text_kv <= n_k entries: the same slot count serves both jobs
  const int groups = fo::ceil_div(static_cast<int64_t>(a.n_q) * a.heads, kRowsPerGroup);
  size_t lds = static_cast<size_t>(kRowsPerGroup) * a.n_k + 8;
  const size_t lds_q = q_job_layout(a.n_q, a.n_k, a.text_kv).bytes;
  if (lds_q > lds) lds = lds_q;
  symbols_kernel<T, E><<<a.batch * (groups + 1), kThreads, lds, stream>>>(a, groups);
  FO_CHECK_LAUNCH();
  return FO_OK;
}

template <typename T, int I = 0>
int dispatch_slots(const ProducerArgs& a, int need, hipStream_t stream) {
  if constexpr (I < static_cast<int>(sizeof(kSlots) / sizeof(kSlots[0]))) {
    if (need <= kSlots[I]) return launch_both<T, kSlots[I]>(a, stream);
    return dispatch_slots<T, I + 1>(a, need, stream);
  } else {
    return fo::fail(FO_ERR_INVALID, "symbols_from_scores: more than %d key blocks", kMaxBlocks);
  }
}

}  // namespace

extern "C" int fo_symbols_from_scores(const void* scores, int dtype, int32_t batch, int32_t num_heads,
                                      int32_t n_q_blocks, int32_t n_kv_blocks, int32_t n_text_q,
                                      int32_t n_text_kv, const float* q_threshold,
                                      const float* kv_threshold, uint8_t* sparse_info,
                                      int32_t* sparse_info_indptr, uint8_t* sparse_kv_info,
                                      int32_t* sparse_kv_info_indptr, void* stream) {
  FO_REQUIRE(dtype == FO_F32 || dtype == FO_BF16 || dtype == FO_F16,
             "symbols_from_scores: scores must be float32, bfloat16 or float16");
  FO_REQUIRE(batch >= 0 && num_heads > 0 && n_q_blocks > 0 && n_kv_blocks > 0,
             "symbols_from_scores: bad sizes batch=%d heads=%d q_blocks=%d kv_blocks=%d", batch,
             num_heads, n_q_blocks, n_kv_blocks);
  FO_REQUIRE(n_kv_blocks <= kMaxBlocks && n_q_blocks <= kMaxBlocks,
             "symbols_from_scores: at most %d blocks per side (got %d x %d)", kMaxBlocks, n_q_blocks,
             n_kv_blocks);
  FO_REQUIRE(n_text_q >= 0 && n_text_q <= n_q_blocks && n_text_kv >= 0 && n_text_kv <= n_kv_blocks,
             "symbols_from_scores: text blocks (%d, %d) outside (%d, %d)", n_text_q, n_text_kv,
             n_q_blocks, n_kv_blocks);
  // the fill step stores image key block j at q block n_text_q + j (test_attn_score.py:58-65)
  FO_REQUIRE(n_text_q + (n_kv_blocks - n_text_kv) <= n_q_blocks,
             "symbols_from_scores: %d image key blocks do not fit behind %d text q blocks in %d q blocks",
             n_kv_blocks - n_text_kv, n_text_q, n_q_blocks);
  const int64_t kv_bytes = (static_cast<int64_t>(n_q_blocks) * num_heads * n_kv_blocks + 7) / 8;
  FO_REQUIRE(kv_bytes * (batch > 0 ? batch : 1) <= INT32_MAX,
             "symbols_from_scores: packed sparse_kv_info exceeds int32 byte offsets");
  if (batch == 0) return FO_OK;
  FO_REQUIRE(scores && q_threshold && kv_threshold && sparse_info && sparse_info_indptr &&
                 sparse_kv_info && sparse_kv_info_indptr,
             "symbols_from_scores: null pointer");
  ProducerArgs a{scores, q_threshold, kv_threshold, sparse_info, sparse_kv_info, sparse_info_indptr,
                 sparse_kv_info_indptr, batch, num_heads, n_q_blocks, n_kv_blocks, n_text_q, n_text_kv};
  const int need = (n_kv_blocks + 63) / 64;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == FO_F32) return dispatch_slots<float>(a, need, s);
  if (dtype == FO_BF16) return dispatch_slots<__hip_bfloat16>(a, need, s);
  return dispatch_slots<__half>(a, need, s);
}
