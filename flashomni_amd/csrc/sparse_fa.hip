// Ragged block-sparse FlashAttention prefill for gfx950 (MI355X), driven by a decoded work list.
//
// One workgroup = 8 wavefronts (512 lanes, two per SIMD) owns one work-list row = one (request,
// 128-row q-block, head).  Wavefront w serves q rows 32*(w%4)..+31 and kv group w/4: the row's
// 64-key tiles are dealt alternately to the two kv groups, each group keeps its own running
// (max, sum, O) state and the two states are merged through LDS when the row ends.  Splitting a
// row over two kv groups halves its latency, which is what bounds the tail when there are only a
// few rows per CU, and gives every SIMD two wavefronts that are kept in opposite phases: one
// feeds the matrix cores (P.V of its previous tile, K.Q^T of its next) while the other runs its
// softmax on the vector ALUs (see the main loop).
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
// K/V tiles go global -> LDS directly (global_load_lds_dwordx4: no staging registers), two LDS
// stages per kv group; K and V of a tile are copied separately, each as soon as its half of a stage
// is free, and their completion is tracked by counting (s_waitcnt vmcnt); two barriers per
// tile.  A wavefront's 64 lanes land on 1 KB of consecutive LDS, so instead of padding the tile
// rows (256 B = 16 chunks of 16 B) are XOR-swizzled: row r keeps logical chunk c at position
// c ^ f(r), f(r) = ((r & 3) << 2) | ((r >> 2) & 3), applied on the global side of the copy.  That
// makes both the row-wise 128-bit K reads (16 consecutive rows, one chunk column) and the 4-row
// transpose reads of V (4 rows x 4 chunks) hit every bank exactly once.
//
// Work distribution: workgroups are persistent and pop rows from 8 queues (one per XCD, chosen by
// blockIdx % 8) that the decoder filled head by head, so one XCD's L2 serves a few heads' K/V; an
// idle XCD steals from its neighbours.  The last workgroup to finish resets the queue cursors.
// When a queue is so short that half of its XCD's workgroups would stay idle, its positions stand
// for parts of rows (ranges of a row's kv blocks): parts publish unnormalised partial results to
// the caller's workspace and the last one to arrive combines them (see the end of the row loop).
//
// Between rows: while kv group 0 combines the two groups' states, one wavefront of group 1 pops the
// next item, gathers its row's metadata and copies its kv block list into LDS, so the next row
// starts with everything at hand: Q (copied into LDS like a K tile, then read as an operand) and
// the first K/V tiles are requested together.  The finished row goes through a padded LDS tile and
// leaves in 16-byte pieces, 16 consecutive lanes per 256-byte output row.  (Both were measured:
// fetched or stored from the accumulator layout, a wavefront instruction is 64 scattered pieces.)
//
// Long lists (eight rows per CU or more) run in a second form of the same kernel: a workgroup is
// 4 wavefronts that own a whole row, two such workgroups share a CU, and the main loop is software-
// pipelined in steps of 32 keys: the MFMAs of S(t+1) and P(t-1).V(t-1) are interleaved, instruction
// by instruction, with the softmax of S(t), the operand reads four slots ahead and the copies two
// steps ahead (see the kPipe branch of the kernel).  Measured on the video-sized lists it is ~5 %
// faster than the two-phase form; on short lists a row's doubled latency costs more than that.
//
// Numerics follow the reference kernel (include/flashomni/attention/prefill.cuh:759-962): base-2
// softmax p = exp2(s*c - m*c) with c = sm_scale*log2(e), P rounded to the activation type before
// P.V, row sum d over the rounded p, O = acc * rcp(d) with one round-to-nearest cast, a row with no
// kv block writes zeros and lse = -5e4 (the finite "infinity" of include/flashomni/math.cuh:32),
// lse = log2(d) + m*c.  Two liberties inside the stated tolerances: for 16-bit inputs c is
// multiplied into Q once per row (one extra rounding of q), and the reference point m is the exact
// row max of the first tile and afterwards raised only when exceeded by more than 2^8.
#include <cstdlib>
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
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

constexpr float kNegInf = -5e4f;  // finite "infinity" of the reference
constexpr int kThreads = 512;
constexpr int kGroupThreads = 256;
constexpr int kBlockQ = 128, kBlockKV = 128, kHeadDim = 128;
constexpr int kTileKV = 64;
constexpr int kRowBytes = 256;   // one K or V row of 128 16-bit elements, unpadded (swizzled)
constexpr int kRowBytes8 = 128;  // one fp8 K row
constexpr int kVBytes = kTileKV * kRowBytes;
constexpr int kMergeOBytes = 4 * 16 * 64 * 16;
constexpr int kOutTileOff = kMergeOBytes + 4 * 64 * 8;  // behind the merge area
constexpr int kOutRowBytes = 256 + 16;                  // one output row of 128 16-bit elements, padded
constexpr int kOutTileBytes = 128 * kOutRowBytes;
// LDS geometry of one kv group: two stages of (K tile, V tile); K is 16-bit or fp8
template <bool kFp8, bool kKLo = false, int kGroups = 2>
struct Geom {
  // (fp8 K with a second term: the tile of k, then the tile of k_lo)
  static constexpr int kKBytes = kTileKV * (kFp8 ? (kKLo ? 2 : 1) * kRowBytes8 : kRowBytes);
  static constexpr int kStageBytes = kKBytes + kVBytes;
  static constexpr int kGroupBytes = 2 * kStageBytes;
  static constexpr int kTilesBytes = kGroups * kGroupBytes;
  // the epilogue reuses the tile buffers: kv group 1's partial O (64 KB fp32) + its (max, sum)
  // pairs (2 KB), then the finished row as a padded tile for the coalesced store (one kv group:
  // no merge area, the output tile starts at 0)
  static constexpr int kOutOff = kGroups == 2 ? kOutTileOff : 0;
  static constexpr int kSmemBytes = kTilesBytes > kOutOff + kOutTileBytes ? kTilesBytes : kOutOff + kOutTileBytes;
};
constexpr int kXcds = 8;
constexpr int kMaxRowBlocks = 4096;  // kv blocks of one row held in LDS (512 Ki tokens per request)
constexpr int kMaxRowBlocksKLo = 2048;  // the same for the two-term k, whose tiles leave less LDS
constexpr int kMaxRowBlocksOneGroup = 3072;  // and for the one-group form (two workgroups share a CU's LDS)
constexpr float kLazyLog2 = 8.0f;  // the running max is raised only past a 2^8 overshoot
// merge area (reuses the tile buffers): O^T of kv group 1, then its (m, d)
static_assert(kOutTileOff + kOutTileBytes <= Geom<true>::kSmemBytes, "merge area must fit");

struct FaParams {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  float* lse;
  const void* q_lo;  // fp8: optional second e4m3 term of q (same layout and scale as q)
  const void* k_lo;  // fp8: optional second e4m3 term of k (same layout and scale as k)
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
  float* split_ws;  // partial results of rows whose kv list is split over workgroups (or null)
  const int32_t* shares;  // even shares: first row of every share, then the rows' cost offsets (or null)
  int32_t num_heads;
  int32_t kv_group;  // q heads per kv head (grouped-query attention); 1 = one kv head per q head
  // 0: a work-list row is (request, 128-token q block, q head).  g > 0: the reference's layout for
  // grouped-query attention with g q heads per kv head (prefill.cuh:410-413, 1283-1290): a row is
  // (request, tile, kv head), the tile being rows tile*128 .. +127 of the request's q tokens x the kv
  // head's g q heads flattened token-major (row r -> token r / g, q head kv_head * g + r % g);
  // row_head holds the kv head and kv_group is 1.
  int32_t gqa_pack;
  int32_t n_q_blocks, n_kv_blocks;  // row lengths of q_scale / k_scale
  float sm_scale_log2;
  // logits soft cap (reference: DefaultAttention, variants.cuh:43-56, :68-70): scores become
  // cap * tanh(q.k * sm_scale / cap).  cap_log2 = cap * log2(e), and sm_scale_log2 then holds
  // 2 * log2(e) * sm_scale / cap, so that exp2 of the scaled product is exp(2x) of tanh's argument.
  float cap_log2;
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
  // acc + sum of the eight elements of v (v_dot2c_f32_bf16 against ones)
  static __device__ __forceinline__ float add_elems(x8 v, float acc) {
    typedef __attribute__((ext_vector_type(2))) __bf16 x2;
    const x2 ones = {static_cast<__bf16>(1.0f), static_cast<__bf16>(1.0f)};
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2_f32_bf16(x2{v[2 * i], v[2 * i + 1]}, ones, acc, false);
    return acc;
  }
};
template <>
struct Types<_Float16> {
  using x8 = f16x8;
  using x4 = f16x4;
  static __device__ __forceinline__ f32x16 mfma(x8 a, x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float add_elems(x8 v, float acc) {
    typedef __attribute__((ext_vector_type(2))) _Float16 x2;
    const x2 ones = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2(x2{v[2 * i], v[2 * i + 1]}, ones, acc, false);
    return acc;
  }
};

typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void glb_void;

// chunk swizzle of a 256-byte LDS tile row r (16 chunks)
__device__ __forceinline__ int swz(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }
// chunk swizzle of a 128-byte LDS tile row r (8 chunks; two rows span the 64 banks)
__device__ __forceinline__ int swz8(int r) { return (r >> 1) & 7; }

// 64 lanes x 16 bytes, global -> LDS: lane i fetches 16 bytes at sbase + voff and lands at LDS byte
// address lds_addr + 16*i.  sbase and lds_addr are wavefront-uniform (scalar registers), so a copy
// costs no vector-ALU work.  Issued as inline assembly on purpose: the compiler then does not
// track the copy, and does not put a vmcnt(0) in front of later LDS reads of the *other* stage that
// it cannot tell apart from the copy's destination (that wait would expose the whole copy latency
// every tile).  All waits on these copies are the explicit s_waitcnt vmcnt(0) + barrier at the
// head of a tile's MFMA block.
__device__ __forceinline__ void copy16_to_lds(const void* sbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(sbase)
               : "memory", "m0");
}

// Four 16-bit values from a 4-row x 16-column LDS patch, transposed across a 16-lane group:
// the group's lane i (0..15) supplies the address of row i/4, columns 4*(i%4)..+3, and receives
// column i of rows 0..3.
__device__ __forceinline__ s16x4 lds_read_tr16(const uint8_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
}

// max of x over lane and lane^32 (v_permlane32_swap: no LDS round trip)
__device__ __forceinline__ float max_across_halves(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const u32x2 r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__builtin_bit_cast(float, r[0]), __builtin_bit_cast(float, r[1]));
}

// words of `sched` (written by the decoder): [0..8] queue bounds inside `order`, [16..23] queue
// cursors, [24] completion counter; [26] even shares in use, [27] cost share of a workgroup, [28]
// total cost, [29] number of shares, [30] number of rows, [31] the share table holds one record per
// queue entry; [64..575] arrival counters of the rows cut at share boundaries
constexpr int kSchedEven = 26, kSchedArrived = 64;
constexpr int kRecordInts = 8;  // queue entry record: row, request, q block, head, first kv slot, kv count
constexpr int kMaxShares = 512, kMaxSplitParts = 4, kRowOverhead = 3;
constexpr int kItemBatch = 16;  // item records of a share gathered at a time
constexpr int kSplitPartFloats = 128 * 128 + 2 * 256;  // O (fp32) + (max, sum) per lane of kv group 0
// Partial results live in 2 * kMaxShares areas of the workspace: share j writes the part of a row
// that began in an earlier share to area 2j and the first part of a row that continues into the
// next share to area 2j + 1 (a share holds at most one of each).
__device__ __forceinline__ int part_area(int first_share, int part) {
  return part == 0 ? 2 * first_share + 1 : 2 * (first_share + part);
}

// Partial results cross workgroups (and XCDs, whose L2s are not coherent with each other) through
// device-scope accesses that bypass the local L2 instead of through fences, which would write back
// and invalidate a whole L2 that is busy serving K and V.
__device__ __forceinline__ void store_pair_device(float* p, float a, float b) {
  const uint64_t v = static_cast<uint64_t>(__float_as_uint(a)) | (static_cast<uint64_t>(__float_as_uint(b)) << 32);
  __hip_atomic_store(reinterpret_cast<uint64_t*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void load_pair_device(const float* p, float& a, float& b) {
  const uint64_t v = __hip_atomic_load(reinterpret_cast<const uint64_t*>(p), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
  a = __uint_as_float(static_cast<uint32_t>(v));
  b = __uint_as_float(static_cast<uint32_t>(v >> 32));
}

// Pop the next row for this workgroup from the queues: own XCD queue first, then the neighbours'.
// `first` is the first queue that may still hold rows: a queue found empty stays empty for the rest
// of the launch, so it is not asked again.  `q` is the launch's copy of the queue bounds: the pop
// itself is one atomic.  Returns the entry's position in `order` or -1.
__device__ __forceinline__ int pop_row(const FaParams& p, int xcd, const int* q, int* first) {
  for (int a = *first; a < kXcds; ++a) {
    const int x = (xcd + a) & (kXcds - 1);
    const int beg = q[x], end = q[x + 1];
    if (beg < end) {
      const int pos = beg + atomicAdd(&p.sched[16 + x], 1);
      if (pos < end) {
        *first = a;
        return pos;
      }
    }
  }
  *first = kXcds;
  return -1;
}

// T: element type of V, P and O (and of Q, K unless kFp8).  kFp8: Q and K are e4m3fn bytes with one
// dequantisation scale per (head, 128-token block); S^T then comes from
// v_mfma_scale_f32_32x32x64_f8f6f4 (64 d per instruction, unit block scale) and the two per-block
// scales are folded into the softmax scale of the tile.  kQLo: q comes as two e4m3 terms, q + q_lo
// (the second one the rounding residual of the first), and S^T = K.(q + q_lo)^T takes two MFMAs
// per slab: e4m3 keeps 3 mantissa bits, and with both operands rounded to it the logits are too
// noisy for the accuracy this path promises; with the two-term q only k's rounding is left.  The
// fp8 matrix cores run at twice the 16-bit rate, so the two terms cost what a 16-bit S^T costs.
// kKLo: k comes as two e4m3 terms as well, k + k_lo; S^T = k.q^T + k.q_lo^T + k_lo.q^T (the product
// of the two residuals, 2^-8 of the logit, is left out): both operands then carry ~7 significant
// bits and the logits are as accurate as 16-bit ones.  This is the accuracy form, not a fast one.
//
// kGroups: kv groups of a workgroup.  2: the form described at the top of this file (8 wavefronts).
// 1: a workgroup is 4 wavefronts (q sub-tiles 0..3) that walk all tiles of the row, two such
// workgroups share a CU (one wavefront of each per SIMD) and run independent rows: nothing ties
// their phases together, there is no merge, and one's row prologue / epilogue overlaps the other's
// main loop.  A row takes twice as long, so this is the form for long lists (many rows per CU).
template <typename T, bool kFp8, bool kQLo, bool kKLo, int kGroups, bool kPipe = false, bool kGqaPack = false,
          bool kCap = false>
__global__ void __launch_bounds__(kGroups * kGroupThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
sparse_fa_kernel(const FaParams p) {
  static_assert(kPipe == (kGroups == 1), "one kv group runs the software-pipelined loop, two the two-phase loop");
  static_assert(!kPipe || !kFp8, "the software-pipelined loop is built for 16-bit operands");
  static_assert(kFp8 || !kQLo, "the two-term q is an fp8 form");
  static_assert(kQLo || !kKLo, "the two-term k is built on the two-term q");
  static_assert(!kCap || (!kFp8 && !kPipe), "the logits soft cap is built into the two-phase loop for 16-bit operands");
  constexpr int kWaves = 4 * kGroups;
  constexpr int kFetchWave = kGroups == 2 ? 4 : 0;  // the wavefront that fetches the next item
  using TT = Types<T>;
  using x8 = typename TT::x8;
  using x4 = typename TT::x4;
  using G = Geom<kFp8, kKLo, kGroups>;
  using TQK = typename std::conditional<kFp8, uint8_t, T>::type;
  constexpr int kStageBytes = G::kStageBytes, kKBytes = G::kKBytes, kGroupBytes = G::kGroupBytes;
  // (256-byte aligned: lane offsets with XOR-swizzled low bits can then carry the array's base)
  extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
  // this item / the next one, with everything the row's prologue needs: fetched by the popping lane
  // while the rest of the workgroup finishes the current row
  struct RowInfo {
    int row, part, parts, slot, req, qb, head, q_begin, q_rows, kv_begin, kv_len, ptr0, nb;
    float q_scale;  // fp8: dequantisation scale of the row's q block
    int k_scale0;   // fp8: position of the request's first kv block in k_scale (the kv head's row)
  };
  // (fetched with the rest of the record: read in the row's prologue, they would wait behind every
  // tile copy in flight)
  auto fill_scales = [&](RowInfo& it) {
    it.q_scale = 1.f;
    it.k_scale0 = 0;
    if constexpr (kFp8) {
      it.q_scale = p.q_scale[static_cast<int64_t>(it.head) * p.n_q_blocks + p.q_blk_base[it.req] + it.qb];
      it.k_scale0 = (it.head / p.kv_group) * p.n_kv_blocks + p.kv_blk_base[it.req];
    }
  };
  // q_begin: first token of the item's q rows; q_rows: how many of its 128 rows exist
  auto set_q_range = [&](RowInfo& it) {
    const int q0 = p.qo_indptr[it.req], q1 = p.qo_indptr[it.req + 1];
    if (kGqaPack) {  // (rows are (token, q head) pairs counted from the request's first token)
      it.q_begin = q0;
      it.q_rows = min(kBlockQ, (q1 - q0) * p.gqa_pack - it.qb * kBlockQ);
    } else {
      it.q_begin = q0 + it.qb * kBlockQ;
      it.q_rows = min(kBlockQ, q1 - it.q_begin);
    }
  };
  __shared__ RowInfo s_next_row[2];
  __shared__ int s_arrived;
  __shared__ int s_queue[16];  // queue bounds and even-share words of `sched`, read once
  __shared__ int s_share[1];   // even shares: items of this workgroup's share handed out so far
  __shared__ int s_guess;      // queues: one past the position this workgroup popped last
  __shared__ RowInfo s_items[kItemBatch];  // even shares: records of the share's next items
  constexpr int kRowBlocks = kGroups == 1 ? kMaxRowBlocksOneGroup : kKLo ? kMaxRowBlocksKLo : kMaxRowBlocks;
  __shared__ uint16_t s_blk2[2][kRowBlocks];  // kv block list of this row / the next one
  // fp8: the k dequantisation scales of the listed blocks (read per tile: from global memory the
  // compiler would wait for every tile copy in flight along with them)
  __shared__ float s_ksc2[2][kFp8 ? kRowBlocks : 1];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);  // wavefront index, kept scalar
  const int qs = wv & 3, kg = wv >> 2;
  const int l32 = lane & 31, g = lane >> 5;
  // The lane index, worked out again where it is called (two instructions) and opaque to the
  // compiler: address terms derived from the kernel-wide `lane` are computed once per launch, find no
  // register across the main loop and come back from scratch memory where they are used.
  auto fresh_lane = [&]() __attribute__((always_inline)) {
    int l = static_cast<int>(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)));
    asm volatile("" : "+v"(l));
    return l;
  };
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

  // The next row is popped by kv group 1 while kv group 0 combines and stores the current one
  // (group 1 has nothing else to do then), so the queue atomics are off the critical path.
  if (tid < 9) s_queue[tid] = p.sched[tid];
  if (tid >= 64 && tid < 64 + 6) s_queue[9 + tid - 64] = p.sched[kSchedEven + tid - 64];
  if (tid == 128) s_guess = 0;
  __syncthreads();
  // Even shares: the decoder has laid the rows out head by head and given every row a cost
  // (kRowOverhead + its kv blocks); share j is the cost range [j * share, (j + 1) * share), and a
  // row that straddles share boundaries is computed in parts by the shares it touches.  Every
  // workgroup holds one share; they are dealt so that the workgroups of one XCD hold neighbouring
  // shares (the same heads' K and V).  A share's items are consecutive rows of `order`, known from
  // the start: their records are gathered sixteen at a time, all in parallel, so that between two
  // rows only the kv block list has to be fetched.
  // (workgroup-uniform words: made scalar, so that none of them occupies a vector register for the
  // whole launch)
  auto queue_word = [&](int i) { return __builtin_amdgcn_readfirstlane(s_queue[i]); };
  const int ev_share = queue_word(10), ev_total = queue_word(11), ev_n = queue_word(12), ev_rows = queue_word(13);
  const bool even = kGroups == 2 && queue_word(9) != 0 && p.shares != nullptr && p.split_ws != nullptr &&
                    static_cast<int>(gridDim.x) == ev_n;
  const int ev_j = (ev_n & (kXcds - 1)) == 0 ? (blockIdx.x & (kXcds - 1)) * (ev_n / kXcds) + blockIdx.x / kXcds
                                             : static_cast<int>(blockIdx.x);
  auto fill_items = [&](int batch_base) {
    const int lane = fresh_lane();
    if (lane < kItemBatch) {
      RowInfo it;
      it.row = -1;
      it.ptr0 = 0;
      it.nb = 0;
      const int a = ev_j * ev_share, b = min(a + ev_share, ev_total);
      const int i = p.shares[ev_j] + batch_base + lane;
      const int32_t* row_start = p.shares + kMaxShares;
      if (a < ev_total && i < ev_rows) {
        const int u = row_start[i], e = row_start[i + 1] - kRowOverhead;  // kv blocks cost [u, e)
        // (a row without kv blocks stands for the last unit of its own overhead)
        if ((e > u ? u : u - 1) < b) {
          const int w = p.order[i];
          it.row = w;
          it.part = 0;
          it.parts = 1;
          it.slot = 0;
          if (e > u) {
            const int j_lo = u / ev_share, j_hi = (e - 1) / ev_share;
            it.part = ev_j - j_lo;
            it.parts = j_hi - j_lo + 1;
            it.slot = j_lo;
          }
          it.req = p.row_req[w];
          it.qb = p.row_qb[w];
          it.head = p.row_head[w];
          set_q_range(it);
          it.kv_begin = p.kv_indptr[it.req];
          it.kv_len = p.kv_indptr[it.req + 1] - it.kv_begin;
          // this share's range of the row's kv blocks
          const int blk_lo = max(a, u) - u, blk_hi = min(min(b, e) - u, kRowBlocks);
          it.ptr0 = p.kv_row_ptr[w] + blk_lo;
          it.nb = max(blk_hi - blk_lo, 0);
          fill_scales(it);
        }
      }
      s_items[lane] = it;
    }
  };
  const bool have_records = queue_word(14) != 0 && p.shares != nullptr;
  int first_queue = 0;  // kept by the popping lane (the first pop is lane 0's, the others lane 256's)
  // One wavefront: lane 0 takes the next item (even shares: from the gathered records; otherwise it
  // pops a row and gathers its metadata, two rounds of loads), then all lanes copy the row's kv
  // block list; both go to LDS for the whole workgroup.
  auto fetch_next = [&](int slot_idx) {
    slot_idx = __builtin_amdgcn_readfirstlane(slot_idx);
    const int lane = fresh_lane();
    RowInfo ri;
    ri.row = -1;
    ri.ptr0 = 0;
    ri.nb = 0;
    if (even) {
      const int c = s_share[0];  // items handed out so far
      if (c > 0 && (c & (kItemBatch - 1)) == 0) fill_items(c);
      if (lane == 0) {
        ri = s_items[c & (kItemBatch - 1)];
        s_share[0] = c + 1;
        s_next_row[slot_idx] = ri;
      }
    } else {
      // Queues.  The trips to memory are kept to two: the pop's atomic travels together with loads of
      // the 64 records that follow this workgroup's last position in the queue (the 32 workgroups of an
      // XCD pop about once per row each, so the answer is nearly always one of them; otherwise the
      // record is read after the pop), and the row's bounds and its kv block list are asked for
      // together once the record is known.
      typedef __attribute__((ext_vector_type(4))) int i32x4;
      const int xcd = blockIdx.x & (kXcds - 1);
      i32x4 w0 = {0, 0, 0, 0}, w1 = w0;  // lane i: the record at queue position win_lo + i
      int win_lo = 0, win_hi = 0;
      if (have_records) {
        const int fq = __builtin_amdgcn_readfirstlane(first_queue);
        if (fq < kXcds) {
          const int x = (xcd + fq) & (kXcds - 1);
          win_lo = max(queue_word(x), __builtin_amdgcn_readfirstlane(s_guess));
          win_hi = min(queue_word(x + 1), win_lo + 64);
          if (win_lo + lane < win_hi) {
            const i32x4* rec = reinterpret_cast<const i32x4*>(p.shares + kMaxShares + kRecordInts * static_cast<int64_t>(win_lo + lane));
            w0 = rec[0];
            w1 = rec[1];
          }
        }
      }
      int at_lane = -1;
      if (lane == 0) at_lane = pop_row(p, xcd, s_queue, &first_queue);
      const int at = __builtin_amdgcn_readfirstlane(at_lane);
      ri.part = 0;
      ri.parts = 1;
      ri.slot = 0;
      if (at >= 0) {
        // (every lane forms the row's values: they are uniform, and lane 0 stores them)
        if (have_records) {
          i32x4 r0, r1;
          if (at >= win_lo && at < win_hi) {
            const int d = at - win_lo;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              r0[j] = __builtin_amdgcn_readlane(w0[j], d);
              r1[j] = __builtin_amdgcn_readlane(w1[j], d);
            }
          } else {
            const i32x4* rec = reinterpret_cast<const i32x4*>(p.shares + kMaxShares + kRecordInts * static_cast<int64_t>(at));
            r0 = rec[0];
            r1 = rec[1];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              r0[j] = __builtin_amdgcn_readfirstlane(r0[j]);
              r1[j] = __builtin_amdgcn_readfirstlane(r1[j]);
            }
          }
          ri.row = r0[0];
          ri.req = r0[1];
          ri.qb = r0[2];
          ri.head = r0[3];
          ri.ptr0 = r1[0];
          ri.nb = min(r1[1], kRowBlocks);
        } else {
          const int w = __builtin_amdgcn_readfirstlane(p.order[at]);
          ri.row = w;
          ri.req = __builtin_amdgcn_readfirstlane(p.row_req[w]);
          ri.qb = __builtin_amdgcn_readfirstlane(p.row_qb[w]);
          ri.head = __builtin_amdgcn_readfirstlane(p.row_head[w]);
          ri.ptr0 = __builtin_amdgcn_readfirstlane(p.kv_row_ptr[w]);
          // (a row longer than the LDS list is cut; the host side refuses such requests at plan time)
          ri.nb = min(__builtin_amdgcn_readfirstlane(p.kv_row_ptr[w + 1]) - ri.ptr0, kRowBlocks);
        }
        // the first 64 entries of the list are asked for before the bounds are waited for
        const int n = ri.nb, list0 = ri.ptr0;
        int blk_first = 0;
        if (lane < n) blk_first = p.kv_idx[list0 + lane];
        set_q_range(ri);
        ri.kv_begin = p.kv_indptr[ri.req];
        ri.kv_len = p.kv_indptr[ri.req + 1] - ri.kv_begin;
        fill_scales(ri);
        if (lane < n) {
          s_blk2[slot_idx][lane] = static_cast<uint16_t>(blk_first);
          if constexpr (kFp8) s_ksc2[slot_idx][lane] = p.k_scale[ri.k_scale0 + blk_first];
        }
        for (int i = 64 + lane; i < n; i += 64) {
          const int blk = p.kv_idx[list0 + i];
          s_blk2[slot_idx][i] = static_cast<uint16_t>(blk);
          if constexpr (kFp8) s_ksc2[slot_idx][i] = p.k_scale[ri.k_scale0 + blk];
        }
      }
      if (lane == 0) {
        s_next_row[slot_idx] = ri;
        if (at >= 0) s_guess = at + 1;
      }
    }
    if (even && __builtin_amdgcn_readfirstlane(ri.row) >= 0) {
      // (even shares: lane 0 holds the item; every lane copies its part of the kv block list)
      const int list0 = __builtin_amdgcn_readfirstlane(ri.ptr0), n = __builtin_amdgcn_readfirstlane(ri.nb);
      const int ks0 = __builtin_amdgcn_readfirstlane(ri.k_scale0);
      for (int i = lane; i < n; i += 64) {
        const int blk = p.kv_idx[list0 + i];
        s_blk2[slot_idx][i] = static_cast<uint16_t>(blk);
        if constexpr (kFp8) s_ksc2[slot_idx][i] = p.k_scale[ks0 + blk];
      }
    }
    // (everything fetched has been used; said explicitly so that the compiler does not carry these
    // loads as pending to the top of the row loop and wait there, behind the previous row's stores)
    __builtin_amdgcn_s_waitcnt(0x0f70);
  };
  if (wv == 0) {
    if (even) {
      if (lane == 0) s_share[0] = 0;
      fill_items(0);
    }
    fetch_next(0);
  }
  for (int row_it = 0;; ++row_it) {
    // s_next_row is published; everyone is done with the previous row's LDS data.  (Not
    // __syncthreads(): its fence would also wait for the row just stored to be acknowledged by
    // memory, a few microseconds that nothing here depends on.)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    const RowInfo& ri = s_next_row[row_it & 1];
    const int w = __builtin_amdgcn_readfirstlane(ri.row);  // uniform values, kept in scalar registers
    if (w < 0) break;
    const int part = __builtin_amdgcn_readfirstlane(ri.part), parts = __builtin_amdgcn_readfirstlane(ri.parts);
    const int split_slot = __builtin_amdgcn_readfirstlane(ri.slot);
    const int req = __builtin_amdgcn_readfirstlane(ri.req), qb = __builtin_amdgcn_readfirstlane(ri.qb);
    const int head = __builtin_amdgcn_readfirstlane(ri.head);
    const int q_begin = __builtin_amdgcn_readfirstlane(ri.q_begin);
    const int q_rows = __builtin_amdgcn_readfirstlane(ri.q_rows);
    const int kv_begin = __builtin_amdgcn_readfirstlane(ri.kv_begin);
    const int kv_len = __builtin_amdgcn_readfirstlane(ri.kv_len);
    const int nb = __builtin_amdgcn_readfirstlane(ri.nb);
    const uint16_t* const s_blk = s_blk2[row_it & 1];

    // (the lane's q row, from a lane index worked out here: see fresh_lane)
    const int lane_p = fresh_lane();
    const int l32_p = lane_p & 31, g_p = lane_p >> 5;
    const int my_row = qs * 32 + l32_p;  // q row of this lane inside the block
    const bool row_ok = my_row < q_rows;
    // row r of the item -> its token (relative to q_begin) and q head (relative to head_q0)
    // (a compile-time variant: as a run-time branch the mapping cost the ungrouped kernel 7 % at the
    // FLUX shape, in how the compiler arranged the code around it)
    const int gq = kGqaPack ? p.gqa_pack : 0;
    const int head_q0 = gq ? head * gq : head;
    auto row_at = [&](int r, int& tok, int& hq) __attribute__((always_inline)) {
      if constexpr (kGqaPack) {
        const uint32_t pr = static_cast<uint32_t>(qb) * kBlockQ + r;
        tok = static_cast<int>(pr / static_cast<uint32_t>(gq));
        hq = static_cast<int>(pr - tok * gq);
      } else {
        tok = r;
        hq = 0;
      }
    };
    // element offset of row r from the item's first q (o) vector, whose strides are sn, sh
    auto row_off = [&](int r, int64_t sn, int64_t sh) __attribute__((always_inline)) {
      int tok, hq;
      row_at(r, tok, hq);
      return tok * sn + hq * sh;
    };
    int my_tok, my_hq;
    row_at(row_ok ? my_row : q_rows - 1, my_tok, my_hq);
    const int64_t q_tok = q_begin + my_tok;
    const int my_head = head_q0 + my_hq;

    if (nb == 0) {
      // listed row without kv blocks: zeros, lse = -5e4
      if (row_ok && kg == 0) {
        T* dst = op + q_tok * p.o_sn + static_cast<int64_t>(my_head) * p.o_sh + g_p * 64;
        const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < 8; ++j) reinterpret_cast<u32x4*>(dst)[j] = z;
        if (p.lse && g_p == 0) p.lse[q_tok * p.num_heads + my_head] = kNegInf;
      }
      if (wv == kFetchWave) fetch_next((row_it + 1) & 1);
      continue;
    }

    f32x16 o_acc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o_acc[dt][i] = 0.f;
    float m_run = 0.f, d_part = 0.f;
    if constexpr (kPipe) {
      // ---- software-pipelined row (one kv group) ----
      // A step is 32 keys.  In step t a wavefront issues the MFMAs of S(t+1) = K(t+1).Q^T and of
      // O^T += V(t-1)^T.P(t-1)^T, and between them, instruction by instruction, the softmax of S(t)
      // (max, exp2, rounding, row sum -> P(t)), the operand reads of later MFMAs and the copies of
      // later steps: the vector ALU work of a step runs in the shadow of its own MFMAs instead of in
      // a phase of its own.  LDS holds four K and four V buffers of 32 keys (8 KB each).  The K
      // operands of a step are read one step ahead (K(t) in step t-2), the V^T operands four slots
      // ahead (V(t) in the second half of step t and the first half of step t+1); a copy is issued as
      // soon as its buffer is dead: K three steps, V two steps before its first read.  One barrier
      // per step.
      constexpr int kStep = 32, kBuf = kStep * kRowBytes;
      // K buffers 0..2 | V buffer 0 | K buffer 3 | V buffers 1..3; Q is staged in the upper 32 KB, so
      // that K(0..2) and V(0) can be requested together with it
      auto kbuf = [&](int i) { return static_cast<uint32_t>(i * kBuf + (i == 3 ? kBuf : 0)); };
      auto vbuf = [&](int i) { return static_cast<uint32_t>((4 + i) * kBuf - (i == 0 ? kBuf : 0)); };
      const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void*)smem));
      const int last_valid = min(kBlockKV, kv_len - s_blk[nb - 1] * kBlockKV);
      const int n_steps = 4 * (nb - 1) + ((last_valid + kStep - 1) / kStep);
      const int kv_head = head / p.kv_group;
      const uint8_t* k_head = reinterpret_cast<const uint8_t*>(
          kp + static_cast<int64_t>(kv_begin) * p.k_sn + static_cast<int64_t>(kv_head) * p.k_sh);
      const uint8_t* v_head = reinterpret_cast<const uint8_t*>(
          vp + static_cast<int64_t>(kv_begin) * p.v_sn + static_cast<int64_t>(kv_head) * p.v_sh);
      // K and V copies go through buffer descriptors that end with the request's last key: a copy
      // that reaches past it (the ragged last 32 keys, or the copies a row's last steps issue for steps
      // that do not exist) touches no memory there, so the loop issues its copies unconditionally.
      // Offsets are 32 bits: the launcher picks this kernel only for kv spans below 4 GiB.
      const uint32_t k_sn2 = static_cast<uint32_t>(p.k_sn) * sizeof(T), v_sn2 = static_cast<uint32_t>(p.v_sn) * sizeof(T);
      const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<uint8_t*>(k_head), 0, static_cast<uint32_t>(kv_len - 1) * k_sn2 + kRowBytes, 0x00020000);
      const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<uint8_t*>(v_head), 0, static_cast<uint32_t>(kv_len - 1) * v_sn2 + kRowBytes, 0x00020000);
      // a lane's part of a copy: row 4 * qs + lane / 16 of a 16-row group, swizzled 16-byte chunk
      uint32_t k_voff = static_cast<uint32_t>(4 * qs + cp_row) * k_sn2 + cp_chunk * static_cast<uint32_t>(sizeof(T));
      uint32_t v_voff = static_cast<uint32_t>(4 * qs + cp_row) * v_sn2 + cp_chunk * static_cast<uint32_t>(sizeof(T));
      asm volatile("" : "+v"(k_voff), "+v"(v_voff));
      const uint32_t m0_base = lds0 + qs * 1024;  // LDS address of this wavefront's part of buffer offset 0
      // 64 lanes x 16 bytes of 4 rows, global -> LDS (see copy16_to_lds), addressed through a descriptor:
      // lane offset + scalar offset
      auto copy_desc = [&](__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff, uint32_t lds_addr) __attribute__((always_inline)) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                     : "memory", "m0");
      };
      auto step_start = [&](int t) { return s_blk[t >> 2] * kBlockKV + (t & 3) * kStep; };
      // the 32 keys of step t (two copy instructions per wavefront) -> their LDS buffer
      auto copy_k = [&](int t) __attribute__((always_inline)) {
        const uint32_t soff = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(step_start(t))) * k_sn2;
#pragma unroll
        for (int j = 0; j < 2; ++j) copy_desc(k_rsrc, k_voff, soff + j * 16 * k_sn2, m0_base + kbuf(t & 3) + j * 4096);
      };
      auto copy_v = [&](int t) __attribute__((always_inline)) {
        const uint32_t soff = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(step_start(t))) * v_sn2;
#pragma unroll
        for (int j = 0; j < 2; ++j) copy_desc(v_rsrc, v_voff, soff + j * 16 * v_sn2, m0_base + vbuf(t & 3) + j * 4096);
      };

      // prologue: Q, K(0..2), V(0) requested together
      {
        const uint8_t* q_head = reinterpret_cast<const uint8_t*>(
            qp + static_cast<int64_t>(q_begin) * p.q_sn + static_cast<int64_t>(head_q0) * p.q_sh);
        const int ln_q = fresh_lane();
        const int cp_row = ln_q >> 4, cp_chunk = ((ln_q & 15) ^ swz(4 * qs + cp_row)) * 8;
#pragma unroll
        for (int n = 0; n < 8; ++n) {
          int r = 4 * (4 * n + qs) + cp_row;
          r = r < q_rows ? r : q_rows - 1;  // ragged last q block: re-read the last row
          copy16_to_lds(q_head, static_cast<uint32_t>((row_off(r, p.q_sn, p.q_sh) + cp_chunk) * sizeof(T)),
                        lds0 + 4 * kBuf + qs * 1024 + n * 4096);
        }
      }
      copy_k(0);
      if (n_steps > 1) copy_k(1);
      if (n_steps > 2) copy_k(2);
      copy_v(0);
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
      __builtin_amdgcn_s_barrier();
      x8 qreg[8], kop[4], vop[4];
      u32x4 pA[2], pB[2];  // P of a step: 2 x 8 rounded values, as 32-bit pairs
      f32x16 sA, sB;
      {
        const int ln_r = fresh_lane();
        const int q_rd_base = (ln_r & 31) * kRowBytes, q_rd_x = ((ln_r >> 5) ^ swz(ln_r & 31)) << 4;
        const uint8_t* qt = smem + 4 * kBuf + qs * 32 * kRowBytes + q_rd_base;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) qreg[ks] = *reinterpret_cast<const x8*>(qt + (q_rd_x ^ (ks << 5)));
        // the softmax scale (log2 domain) is folded into Q, so S^T needs no multiply
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
#pragma unroll
          for (int e = 0; e < 8; ++e) qreg[ks][e] = static_cast<T>(static_cast<float>(qreg[ks][e]) * c);
      }
      // LDS address of the K operand reads of a step, without the buffer's offset (an immediate of the
      // read): read i is at kx0 ^ (i << 5) (row bits, chunk bits and the 256-byte aligned base of
      // the array do not overlap)
      typedef __attribute__((address_space(3))) const x8 lds_x8;
      uint32_t kx0 = lds0 + static_cast<uint32_t>(k_rd_base | k_rd_x);
      asm volatile("" : "+v"(kx0));
      // K operand slice i (16 d) of the step whose K is in buffer `buf`
      auto read_k = [&](uint32_t kx, int buf, int i) __attribute__((always_inline)) {
        return *reinterpret_cast<lds_x8*>(static_cast<uintptr_t>((kx ^ (i << 5)) + kbuf(buf)));
      };
      // the same for the V^T operand reads: the eight lane offsets with the array's base added
      uint32_t vrd[4][2];
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int hi = 0; hi < 2; ++hi) {
          vrd[dt][hi] = lds0 + static_cast<uint32_t>(v_rd_off[dt][hi]);
          asm volatile("" : "+v"(vrd[dt][hi]));
        }
      // V^T operand (kk, dt) of the step whose V is in buffer `buf`: 16 keys x 32 d, transposed
      auto read_v = [&](int buf, int kk, int dt) __attribute__((always_inline)) {
        union {
          s16x4 h[2];
          x8 v;
        } a;
        const uint32_t off = vbuf(buf) + kk * 16 * kRowBytes;
        a.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_s16x4*>(static_cast<uintptr_t>(vrd[dt][0] + off)));
        a.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_s16x4*>(static_cast<uintptr_t>(vrd[dt][1] + off)));
        return a.v;
      };
#pragma unroll
      for (int i = 0; i < 16; ++i) sA[i] = 0.f;
      {
        x8 k0[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) k0[i] = read_k(kx0, 0, i);
#pragma unroll
        for (int i = 0; i < 8; ++i) sA = TT::mfma(k0[i], qreg[i], sA);
      }
      __builtin_amdgcn_sched_barrier(0);
      // (a row of one step reads a buffer nobody filled: the result is never used)
#pragma unroll
      for (int i = 0; i < 4; ++i) kop[i] = read_k(kx0, 1, i);
      // (a row's first step multiplies P(-1) = 0 by what vop holds and by what its first half reads
      // from V buffer 3, where Q was staged: both must be finite whatever Q holds)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) vop[i][e] = static_cast<T>(0.f);
#pragma unroll
      for (int e = 0; e < 4; ++e) pA[0][e] = pA[1][e] = pB[0][e] = pB[1][e] = 0u;
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): Q and K(0) are in registers
      __builtin_amdgcn_s_barrier();        // ... of every wavefront: their LDS space is free
      {
        // V buffer 3 (read by the first step as "V(-1)"), and for a row of fewer than four steps
        // every V buffer it does not fill (read by its padded steps), must not hold Q any more
        const u32x4 z = {0u, 0u, 0u, 0u};
        for (int b = min(n_steps, 3); b < 4; ++b) {
          u32x4* vb = reinterpret_cast<u32x4*>(smem + vbuf(b));
          vb[tid] = z;
          vb[tid + kGroupThreads] = z;
        }
      }
      if (n_steps > 1) {
        copy_v(1);
        copy_k(min(3, n_steps - 1));  // (kept to four instructions per group: the loop's waits count them)
      }

#pragma unroll
      for (int i = 0; i < 16; ++i) sB[i] = 0.f;  // S(1) accumulates from the reference point 0, moved by the first step
      // Block numbers of the row's list as scalars: blk0 = the block of the current four steps, blk1
      // the one after it.  They come from a register that holds 64 consecutive entries of the list,
      // one per lane, refilled every 64 blocks: the loop itself reads no list from LDS (the wait
      // for such a read would also wait for the operand reads in flight).
      int blk_win = s_blk[min(lane, nb - 1)];
      int blk0 = 0, blk1 = 0;
      typedef __attribute__((ext_vector_type(2))) T x2;
      const x2 ones2 = {static_cast<T>(1.0f), static_cast<T>(1.0f)};
      // One step (kB = t % 4 picks the LDS buffers).  Straight-line code apart from small
      // wavefront-uniform branches, so that the accumulators stay where they are.  Eight slots, each:
      // one MFMA of S(t+1), one K operand read of step t+2, one MFMA of P(t-1).V(t-1), the V^T operand
      // needed four slots later, and the softmax of two values of S(t): exp2, rounding, row sum; the
      // accumulator that held them is set to the reference point for its next use (S(t+2)
      // accumulates onto -m_run, so that p = exp2(S) with no subtraction).
      auto do_step = [&](int t, auto buf_tag, f32x16& s_cur, f32x16& s_next, u32x4 (&p_prev)[2], u32x4 (&p_cur)[2]) __attribute__((always_inline)) {
        constexpr int kB = decltype(buf_tag)::value;
        // V(t) and K(t+2), first read in this step, were requested two barriers ago: they have landed
        // once only the four copies of the last barrier are outstanding; after the barrier that holds
        // for every wavefront
        __builtin_amdgcn_s_waitcnt(0x0f70 | 4);  // vmcnt(4)
        // (the buffers that this step's copies overwrite were last read in the first half of step t-1:
        // the twelve operand reads of its second half may still be in flight)
        __builtin_amdgcn_s_waitcnt(0xcc7f);  // lgkmcnt(12)
        __builtin_amdgcn_s_barrier();
        // this step's copies: V(t+2) into the buffer of V(t-2) and K(t+4) into the buffer of K(t), both
        // last read in step t-1.  Their scalar offsets are worked out here from the block numbers held
        // in scalar registers; the four instructions go out between the MFMAs below (V first, then
        // K).  Steps past the row's end copy a block again or nothing (see the descriptors).
        const uint32_t v_soff = static_cast<uint32_t>(((kB + 2) < 4 ? blk0 : blk1) * kBlockKV + ((kB + 2) & 3) * kStep) * v_sn2;
        const uint32_t k_soff = static_cast<uint32_t>(blk1 * kBlockKV + kB * kStep) * k_sn2;
        // (a row is padded to a multiple of four steps; a padded step has no keys: p = 0, against V
        // operands read from buffers that hold earlier steps of the same row)
        const int valid = t < n_steps ? min(kStep, kv_len - (blk0 * kBlockKV + kB * kStep)) : 0;
        if (valid < kStep) {
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int kv = (i >> 2) * 8 + g * 4 + (i & 3);
            if (kv >= valid) s_cur[i] = -INFINITY;  // p = 0
          }
        }
        float mx = s_cur[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s_cur[i]);
        mx = max_across_halves(mx);  // row max relative to m_run
        const bool first = t == 0;
        // The reference point moves always on a row's first step, afterwards only past a 2^8
        // overshoot (a rare, wavefront-uniform branch that changes registers in place): S(t), the
        // accumulator of S(t+1), which holds the old point, and the row sum move now; O, which still
        // receives P(t-1).V(t-1) at the old point in this step, is rescaled at the step's end.
        const bool moved = first || __builtin_expect(__any(mx > kLazyLog2), 0);
        float o_scale = 1.f;
        if (moved) {
          const float delta = first ? mx : fmaxf(mx, 0.f);
          if (!first) {
            o_scale = __builtin_amdgcn_exp2f(-delta);
            d_part *= o_scale;
          }
          m_run += delta;
#pragma unroll
          for (int i = 0; i < 16; ++i) s_cur[i] -= delta;
#pragma unroll
          for (int i = 0; i < 16; ++i) s_next[i] -= delta;
        }
        const f32x2 neg_m2 = {-m_run, -m_run};
        // (made opaque once per step: otherwise the eight read offsets are worked out once per
        // kernel and live in eight registers, which the loop does not have)
        uint32_t kx = kx0;
        asm volatile("" : "+v"(kx));
        float psum = 0.f;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          s_next = TT::mfma(kop[i & 3], qreg[i], s_next);
          // the operand of the S MFMA four slots on: second half of K(t+1), then first half of K(t+2)
          kop[i & 3] = i < 4 ? read_k(kx, (kB + 1) & 3, i + 4) : read_k(kx, (kB + 2) & 3, i - 4);
          o_acc[i & 3] = TT::mfma(vop[i & 3], __builtin_bit_cast(x8, p_prev[i >> 2]), o_acc[i & 3]);
          // the operand of the P.V MFMA four slots on: second half of V(t-1), then first half of V(t)
          vop[i & 3] = i < 4 ? read_v((kB + 3) & 3, 1, i) : read_v(kB, 0, i - 4);
          // (the two values are pinned to this slot: without the empty statements the compiler
          // gathers all exponentials of a step in front of its MFMAs)
          float e0 = s_cur[2 * i], e1 = s_cur[2 * i + 1];
          asm volatile("" : "+v"(e0), "+v"(e1));
          const x2 pk = {static_cast<T>(__builtin_amdgcn_exp2f(e0)), static_cast<T>(__builtin_amdgcn_exp2f(e1))};
          uint32_t pu = __builtin_bit_cast(uint32_t, pk);
          // the row sum is taken over the rounded p, as the reference does
          if constexpr (std::is_same<T, __bf16>::value) {
            psum = __builtin_amdgcn_fdot2_f32_bf16(pk, ones2, psum, false);
          } else {
            psum = __builtin_amdgcn_fdot2(pk, ones2, psum, false);
          }
          // (the accumulator that held the two values is set to the reference point for its next use)
          f32x2 r01 = neg_m2;
          asm volatile("" : "+v"(pu), "+v"(psum), "+v"(r01));
          p_cur[i >> 2][i & 3] = pu;
          s_cur[2 * i] = r01[0];
          s_cur[2 * i + 1] = r01[1];
          if (i == 1 || i == 3) {
            copy_desc(v_rsrc, v_voff, v_soff + (i >> 1) * 16 * v_sn2, m0_base + vbuf((kB + 2) & 3) + (i >> 1) * 4096);
          } else if (i == 5 || i == 7) {
            copy_desc(k_rsrc, k_voff, k_soff + ((i - 4) >> 1) * 16 * k_sn2, m0_base + kbuf(kB) + ((i - 4) >> 1) * 4096);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        d_part += psum;
        if (moved && !first) {
#pragma unroll
          for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o_acc[dt][i] *= o_scale;
        }
      };
      using B0 = std::integral_constant<int, 0>;
      using B1 = std::integral_constant<int, 1>;
      using B2 = std::integral_constant<int, 2>;
      using B3 = std::integral_constant<int, 3>;
      for (int t = 0; t < n_steps; t += 4) {
        const int bi = t >> 2;
        blk0 = __builtin_amdgcn_readlane(blk_win, bi & 63);
        if (((bi + 1) & 63) == 0) blk_win = s_blk[min(bi + 1 + lane, nb - 1)];
        blk1 = __builtin_amdgcn_readlane(blk_win, (bi + 1) & 63);
        do_step(t, B0{}, sA, sB, pB, pA);
        do_step(t + 1, B1{}, sB, sA, pA, pB);
        do_step(t + 2, B2{}, sA, sB, pB, pA);
        do_step(t + 3, B3{}, sB, sA, pA, pB);
      }
      // P.V of the last step (real or padded; its V is in buffer 3, vop holds the first half)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        o_acc[i] = TT::mfma(vop[i], __builtin_bit_cast(x8, pB[0]), o_acc[i]);
        vop[i] = read_v(3, 1, i);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) o_acc[i] = TT::mfma(vop[i], __builtin_bit_cast(x8, pB[1]), o_acc[i]);
      // The copies of the steps past the row's end (the loop asks for K four and V two steps ahead,
      // whatever is left of the row) are still in flight: they must have landed before the epilogue
      // lays the finished row out in the same LDS.  (Nothing else waits for them: the barrier below
      // orders LDS accesses, not these copies, which the compiler does not see.)
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    } else {
    // Q operand.  A lane needs q row l32 of its sub-tile, 16 bytes out of every 32 (fp8: 32 of 64):
    // fetched straight from memory that is 64 scattered pieces per instruction (measured: ~4 k
    // cycles per row).  The 128 q rows are copied into LDS like a K tile instead (64 rows per kv
    // group, into the V half of its stage 1, which is free until the first MFMA block) and read
    // from there.  Requested first so that the latency overlaps the staging below.
    x8 qreg[kFp8 ? 1 : 8];
    i32x8 qreg8[kFp8 ? 2 : 1];
    i32x8 qlo8[kQLo ? 2 : 1];
    const uint32_t lds_group = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void*)group_smem));
    if constexpr (kFp8) {
      // (fp8 Q, half the bytes, is still fetched directly: with the LDS detour hipcc arranges the
      // main loop of this instantiation less well, which costs more than the detour saves)
      const uint8_t* src = qp + q_tok * p.q_sn + static_cast<int64_t>(my_head) * p.q_sh + g_p * 32;
#pragma unroll
      for (int sl = 0; sl < 2; ++sl) {
        const i32x4 lo = *reinterpret_cast<const i32x4*>(src + sl * 64);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(src + sl * 64 + 16);
        qreg8[sl] = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
      if constexpr (kQLo) {
        const uint8_t* src2 = static_cast<const uint8_t*>(p.q_lo) + q_tok * p.q_sn +
                              static_cast<int64_t>(my_head) * p.q_sh + g_p * 32;
#pragma unroll
        for (int sl = 0; sl < 2; ++sl) {
          const i32x4 lo = *reinterpret_cast<const i32x4*>(src2 + sl * 64);
          const i32x4 hi = *reinterpret_cast<const i32x4*>(src2 + sl * 64 + 16);
          qlo8[sl] = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
      }
    } else {
      const uint8_t* q_head = reinterpret_cast<const uint8_t*>(
          qp + static_cast<int64_t>(q_begin) * p.q_sn + static_cast<int64_t>(head_q0) * p.q_sh);
      const uint32_t qdst = lds_group + kStageBytes + kKBytes + qs * 1024;
      const int ln_q = fresh_lane();
      const int cp_row = ln_q >> 4, cp_chunk = ((ln_q & 15) ^ swz(4 * qs + cp_row)) * 8;
#pragma unroll
      for (int n = 0; n < 4; ++n) {
        int r = kg * 64 + 4 * (4 * n + qs) + cp_row;
        r = r < q_rows ? r : q_rows - 1;  // ragged last q block: re-read the last row
        copy16_to_lds(q_head, static_cast<uint32_t>((row_off(r, p.q_sn, p.q_sh) + cp_chunk) * sizeof(T)),
                      qdst + n * 4096);
      }
    }
    // (the row's kv block list is in LDS already: the main loop has no global loads besides the
    // tile copies, whose completion it tracks by counting, s_waitcnt vmcnt)
    // number of 64-key tiles; only the last listed block can be the request's ragged tail
    int n_tiles = 2 * nb;
    if (kv_len - s_blk[nb - 1] * kBlockKV <= kTileKV) n_tiles -= 1;
    const int my_tiles = (n_tiles - kg + 1) >> 1;  // tiles kg, kg+2, ...

    // softmax scale in the log2 domain; with fp8 operands the per-block dequantisation scales of
    // q (one per row of the list) and k (one per kv block) are folded in tile by tile
    float cq = c;
    if constexpr (kFp8) cq *= __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, ri.q_scale)));
    const int kv_head = head / p.kv_group;
    const float* const s_ksc = s_ksc2[row_it & 1];

    // Running reference point m_run of the softmax (log2 domain), partial sum d_part.  S^T is formed
    // relative to m_run: the MFMA accumulator starts at -m_run (c_init), so p = exp2(S^T) directly.
    // m_run is set to the tile's exact row max on the first tile and afterwards only raised when a
    // row's new max exceeds it by more than kLazyLog2 (p then stays <= 2^kLazyLog2, harmless in
    // fp32 / bf16 / fp16): the rescale of O leaves the steady-state path.
    f32x16 c_init;
#pragma unroll
    for (int i = 0; i < 16; ++i) c_init[i] = 0.f;

    // Tile copies.  The address of a copy is a wavefront-uniform tile base plus a per-lane byte
    // offset that does not change from tile to tile (row inside the tile, swizzled chunk); only a
    // request's ragged last tile clamps rows.  Tile j of this kv group = 64 keys of block j of the
    // row's list; it lives in LDS stage j & 1.  K and V of a tile are copied at different times,
    // each as early as its half of the stage is free:
    //   K of tile j+2 at the start of the VALU block of tile j   (K of tile j was consumed by S(j))
    //   V of tile j+1 during the MFMA block of tile j            (V of tile j-1 is in registers)
    // so a K copy has about two block periods to land and a V copy more than one.
    const TQK* k_head = kp + static_cast<int64_t>(kv_begin) * p.k_sn + static_cast<int64_t>(kv_head) * p.k_sh;
    const T* v_head = vp + static_cast<int64_t>(kv_begin) * p.v_sn + static_cast<int64_t>(kv_head) * p.v_sh;
    // lane offsets of copy instruction 0; instruction n adds a uniform 16 (fp8 K: 32) rows
    const uint32_t v_voff = static_cast<uint32_t>((4 * qs + cp_row) * p.v_sn + cp_chunk) * sizeof(T);
    const uint32_t k_voff = kFp8 ? static_cast<uint32_t>((8 * qs + cp8_row) * p.k_sn + cp8_chunk)
                                 : static_cast<uint32_t>((4 * qs + cp_row) * p.k_sn + cp_chunk) * sizeof(T);
    const int64_t k_jstep = (kFp8 ? 32 : 16) * p.k_sn * static_cast<int64_t>(sizeof(TQK));
    const int64_t v_jstep = 16 * p.v_sn * static_cast<int64_t>(sizeof(T));
    constexpr int kKCopies = (kFp8 && !kKLo) ? 2 : 4, kVCopies = 4;  // copy instructions per wavefront and tile
    const uint8_t* klo_head = nullptr;
    if constexpr (kKLo)
      klo_head = static_cast<const uint8_t*>(p.k_lo) + static_cast<int64_t>(kv_begin) * p.k_sn +
                 static_cast<int64_t>(kv_head) * p.k_sh;
    auto tile_start = [&](int j) { return s_blk[j] * kBlockKV + kg * kTileKV; };
    auto tile_valid = [&](int j) { return min(kTileKV, kv_len - tile_start(j)); };
    // all K copies of tile j at once
    auto copy_k = [&](int j) {
      const int start = __builtin_amdgcn_readfirstlane(tile_start(j));
      const int valid = min(kTileKV, kv_len - start);
      const uint8_t* kt = reinterpret_cast<const uint8_t*>(k_head + static_cast<int64_t>(start) * p.k_sn);
      const uint32_t kdst = lds_group + (j & 1) * kStageBytes + qs * 1024;
      // (two-term k: copy instructions 0, 1 fetch the tile of k, 2, 3 that of k_lo behind it)
      constexpr int kPerTerm = kKLo ? 2 : kKCopies;
      const uint8_t* kt_lo = kKLo ? klo_head + static_cast<int64_t>(start) * p.k_sn : nullptr;
      if (__builtin_expect(valid == kTileKV, 1)) {
#pragma unroll
        for (int n = 0; n < kKCopies; ++n)
          copy16_to_lds((n < kPerTerm ? kt : kt_lo) + (n % kPerTerm) * k_jstep, k_voff, kdst + n * 4096);
      } else {
        // ragged tail: re-read the last valid row, never overrun
        const int ln_c = fresh_lane();
        const int cp_row = ln_c >> 4, cp_chunk = ((ln_c & 15) ^ swz(4 * qs + cp_row)) * 8;
        const int cp8_row = ln_c >> 3, cp8_chunk = ((ln_c & 7) ^ ((4 * (qs & 1) + (ln_c >> 4)) & 7)) * 16;
#pragma unroll
        for (int n = 0; n < kKCopies; ++n) {
          int r = (kFp8 ? 8 : 4) * (4 * (n % kPerTerm) + qs) + (kFp8 ? cp8_row : cp_row);
          r = r < valid ? r : valid - 1;
          const uint32_t off = kFp8 ? static_cast<uint32_t>(r * p.k_sn + cp8_chunk)
                                    : static_cast<uint32_t>((r * p.k_sn + cp_chunk) * sizeof(T));
          copy16_to_lds(n < kPerTerm ? kt : kt_lo, off, kdst + n * 4096);
        }
      }
    };
    // V copies of tile j: prepared once, then issued one instruction at a time between MFMAs (a
    // wavefront that issues its share in one burst sits in the issue stage while the CU's address
    // unit, 64 B/clk, works through the burst of all eight wavefronts)
    const uint8_t* cp_v = nullptr;
    uint32_t cp_vdst = 0;
    bool cp_pending = false;
    int cp_valid = kTileKV;
    // scalar part (any time: it touches no LDS stage)
    auto copy_v_address = [&](int j) {
      const int start = __builtin_amdgcn_readfirstlane(tile_start(j));
      cp_valid = min(kTileKV, kv_len - start);
      cp_v = reinterpret_cast<const uint8_t*>(v_head + static_cast<int64_t>(start) * p.v_sn);
      cp_vdst = lds_group + (j & 1) * kStageBytes + kKBytes + qs * 1024;
    };
    // once the target stage is free: arm the one-by-one issue, or issue a ragged tile at once
    auto copy_v_prepare = [&]() {
      const int valid = cp_valid;
      cp_pending = valid == kTileKV;
      if (__builtin_expect(!cp_pending, 0)) {
        const int ln_c = fresh_lane();
        const int cp_row = ln_c >> 4, cp_chunk = ((ln_c & 15) ^ swz(4 * qs + cp_row)) * 8;
#pragma unroll
        for (int n = 0; n < kVCopies; ++n) {
          int r = 4 * (4 * n + qs) + cp_row;
          r = r < valid ? r : valid - 1;
          copy16_to_lds(cp_v, static_cast<uint32_t>((r * p.v_sn + cp_chunk) * sizeof(T)), cp_vdst + n * 4096);
        }
      }
    };
    auto copy_v_issue = [&](int n) {
      if (cp_pending) copy16_to_lds(cp_v + n * v_jstep, v_voff, cp_vdst + n * 4096);
    };
    // wait until at most n of this wavefront's copy instructions are outstanding (they complete in
    // issue order, so "the copies issued after X" outstanding means X has landed)
    auto wait_copies = [&](int n) {
      if (n >= 8) {
        __builtin_amdgcn_s_waitcnt(0x0f70 | 8);
      } else if (n >= 6) {
        __builtin_amdgcn_s_waitcnt(0x0f70 | 6);
      } else if (n >= 4) {
        __builtin_amdgcn_s_waitcnt(0x0f70 | 4);
      } else {
        __builtin_amdgcn_s_waitcnt(0x0f70);
      }
    };

    // ---- main loop: two-phase ("ping-pong") schedule ----
    // A wavefront alternates between an MFMA block (P.V of the previous tile, then K.Q^T of the
    // next) and a VALU block (online softmax).  The two kv groups share the SIMDs (wavefront w and
    // w+4 sit on SIMD w%4) and run half a period apart: every block starts at a workgroup barrier
    // and kv group 1 takes one extra barrier up front, so while one group's wavefronts feed the
    // matrix cores the other group's run their softmax on the vector ALUs.
    //   barrier calls: group 0 makes 2*T0 + 1, group 1 makes 1 + 2*T1 + 1 (T = tiles of the group);
    //   both pad to the larger count before the merge.
    const int calls_mine = kg == 0 ? 2 * ((n_tiles + 1) >> 1) + 1 : 2 * (n_tiles >> 1) + 2;
    const int calls_all = max(2 * ((n_tiles + 1) >> 1) + 1, 2 * (n_tiles >> 1) + 2);
    // copy order of a wavefront: K0, V0, K1 | V1 (MFMA block 0) | K2 (VALU block 0) | V2 | K3 | ...
    if (my_tiles > 0) {
      copy_k(0);
      copy_v_address(0);
      copy_v_prepare();
#pragma unroll
      for (int n = 0; n < kVCopies; ++n) copy_v_issue(n);
      cp_pending = false;
      if (my_tiles > 1) {
        copy_k(1);
        copy_v_address(1);
      }
    }
    // Q has landed once only the tile copies issued after it are outstanding; then for every
    // wavefront after the barrier
    if constexpr (!kFp8) {
      if (my_tiles > 1) {
        __builtin_amdgcn_s_waitcnt(0x0f70 | (2 * kKCopies + kVCopies));
      } else if (my_tiles == 1) {
        __builtin_amdgcn_s_waitcnt(0x0f70 | (kKCopies + kVCopies));
      } else {
        __builtin_amdgcn_s_waitcnt(0x0f70);
      }
    }
    __builtin_amdgcn_s_barrier();
    // Q from LDS while the first tile copies are in flight: rows (qs % 2) * 32 + l32 of the tile that
    // kv group qs / 2 copied, addressed like a K operand
    if constexpr (!kFp8) {
      // (the lane terms are made opaque here: otherwise the eight read addresses are worked out once
      // per kernel, live across the main loop, and their reloads wait for every copy in flight)
      const int ln_r = fresh_lane();
      const int q_rd_base = (ln_r & 31) * kRowBytes, q_rd_x = ((ln_r >> 5) ^ swz(ln_r & 31)) << 4;
      const uint8_t* qt = smem + (qs >> 1) * kGroupBytes + kStageBytes + kKBytes + (qs & 1) * 32 * kRowBytes +
                          q_rd_base;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) qreg[ks] = *reinterpret_cast<const x8*>(qt + (q_rd_x ^ (ks << 5)));
      // the softmax scale (log2 domain) is folded into Q, so S^T needs no multiply
#pragma unroll
      for (int ks = 0; ks < 8; ++ks)
#pragma unroll
        for (int e = 0; e < 8; ++e) qreg[ks][e] = static_cast<T>(static_cast<float>(qreg[ks][e]) * c);
    }
    // (every wavefront holds its Q before the first barrier: the V copies of tile 1 overwrite it after)
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    if (kg == 1) __builtin_amdgcn_s_barrier();

    f32x16 s[2];
    x8 vop[4][4], pb[4];

    // K operand reads of stage `it & 1`, d slices ks0..ks0+3 of both 32-key halves (16-bit K):
    // kop[h][ks - ks0] = rows h*32 + l32, d = ks*16 + g*8 .. +7
    auto read_k = [&](int it, int ks0, x8 (&kop)[2][4]) {
      const uint8_t* ks_base = group_smem + (it & 1) * kStageBytes + k_rd_base;
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int h = 0; h < 2; ++h)
          kop[h][j] = *reinterpret_cast<const x8*>(ks_base + h * 32 * kRowBytes + (k_rd_x ^ ((ks0 + j) << 5)));
    };
    // four d slices of S^T for both 32-key halves; the two accumulator chains alternate so that no
    // MFMA waits for the one issued just before it
    auto s_math = [&](int ks0, const x8 (&kop)[2][4], int j0) {  // d slices ks0+j0, ks0+j0+1
#pragma unroll
      for (int j = j0; j < j0 + 2; ++j)
#pragma unroll
        for (int h = 0; h < 2; ++h)
          s[h] = TT::mfma(kop[h][j], qreg[ks0 + j], (ks0 + j) == 0 ? c_init : s[h]);
    };
    // fp8: S^T straight from LDS (four reads, four MFMAs)
    auto s_fp8 = [&](int it) {
      if constexpr (kFp8) {
        const uint8_t* ks_base = group_smem + (it & 1) * kStageBytes;
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
        for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
          for (int i = 0; i < 16; ++i) s[mt][i] = 0.f;
#pragma unroll
          for (int sl = 0; sl < 2; ++sl)
            s[mt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(k8[mt][sl], qreg8[sl], s[mt], 0, 0, 0,
                                                                    0x7f7f7f7f, 0, 0x7f7f7f7f);
        }
        if constexpr (kQLo) {
          // (second pass so that the two accumulator chains keep alternating)
#pragma unroll
          for (int sl = 0; sl < 2; ++sl)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
              s[mt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(k8[mt][sl], qlo8[sl], s[mt], 0, 0, 0,
                                                                      0x7f7f7f7f, 0, 0x7f7f7f7f);
        }
        if constexpr (kKLo) {
          // k_lo . q^T: the tile of k_lo sits behind the tile of k in the stage
#pragma unroll
          for (int sl = 0; sl < 2; ++sl)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
              const uint8_t* rowp = ks_base + kTileKV * kRowBytes8 + mt * 32 * kRowBytes8 + k_rd_base;
              const i32x4 lo = *reinterpret_cast<const i32x4*>(rowp + (k_rd_x ^ (sl << 6)));
              const i32x4 hi = *reinterpret_cast<const i32x4*>(rowp + ((k_rd_x ^ (sl << 6)) ^ 16));
              const i32x8 kl = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
              s[mt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kl, qreg8[sl], s[mt], 0, 0, 0,
                                                                      0x7f7f7f7f, 0, 0x7f7f7f7f);
            }
        }
      }
    };
    // O^T += V^T . P^T for 16-key slabs kk0, kk0+1
    auto pv_math = [&](int kk) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) o_acc[dt] = TT::mfma(vop[kk][dt], pb[kk], o_acc[dt]);
    };
    // VALU block of tile `it`: all V^T operands of the tile (4 slabs of 16 keys x 4 d tiles) are
    // requested first and land during the softmax
    auto valu_block = [&](int it, bool first) {
      // V of tile `it` has landed once only the copies issued after it (K and V of tile it+1) are
      // outstanding; after the barrier that holds for the whole kv group, and the group is done
      // reading K of this stage, which tile it+2 may now overwrite
      __builtin_amdgcn_s_setprio(0);
      wait_copies(it + 1 < my_tiles ? kKCopies + kVCopies : 0);
      __builtin_amdgcn_s_barrier();
      if (it + 2 < my_tiles) copy_k(it + 2);
      const int valid = tile_valid(it);
      float cs = cq;
      if constexpr (kFp8) cs = cq * s_ksc[it];
      const uint8_t* vs_base = group_smem + (it & 1) * kStageBytes + kKBytes;
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
      // online softmax (per lane: one q column, 32 kv values), log2 domain.  s holds x - m_run
      // (fp8: raw dot products, scaled and shifted here because the scale changes per kv block)
      if constexpr (kFp8) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) s[mt][i] = __builtin_fmaf(s[mt][i], cs, -m_run);
      }
      if constexpr (kCap) {
        // s holds 2 x log2(e) of tanh's argument x (the accumulators start at zero here):
        // tanh(x) = 1 - 2 / (1 + exp(2x)); score = cap_log2 * tanh(x), taken relative to m_run
        const float a = -2.f * p.cap_log2, b = p.cap_log2 - m_run;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i)
            s[mt][i] = __builtin_fmaf(__builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(s[mt][i])), a, b);
      }
      if (valid < kTileKV) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int kv = mt * 32 + (i >> 2) * 8 + g * 4 + (i & 3);
            if (kv >= valid) s[mt][i] = -INFINITY;  // p = 0
          }
      }
      float mx = s[0][0];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[mt][i]);
      mx = max_across_halves(mx);  // row max relative to m_run
      if (first || __builtin_expect(__any(mx > kLazyLog2), 0)) {
        const float delta = first ? mx : fmaxf(mx, 0.f);
        if (!first) {
          const float scale = __builtin_amdgcn_exp2f(-delta);
          d_part *= scale;
#pragma unroll
          for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o_acc[dt][i] *= scale;
        }
        m_run += delta;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) s[mt][i] -= delta;
        if constexpr (!kCap) {
#pragma unroll
          for (int i = 0; i < 16; ++i) c_init[i] = -m_run;
        }
      }
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          pb[mt * 2 + (i >> 3)][i & 7] = static_cast<T>(__builtin_amdgcn_exp2f(s[mt][i]));
      // the row sum is taken over the rounded p, as the reference does
      float psum = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) psum = TT::add_elems(pb[j], psum);
      d_part += psum;
      if (it + 2 < my_tiles) copy_v_address(it + 2);  // for the V copies of the next MFMA block
      __builtin_amdgcn_sched_barrier(0);
    };
    // start of an MFMA block: K of tile `it` has landed once only the copies issued after it (V of
    // this tile, K of the next) are outstanding, and this wavefront's V^T reads of the previous tile
    // have returned; after the barrier both hold for the whole kv group, so the V half of the other
    // stage may be overwritten
    auto open_mfma_block = [&](int it) {
      wait_copies(kVCopies + (it + 1 < my_tiles ? kKCopies : 0));
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_s_setprio(3);  // the MFMA block outranks the other kv group's softmax at issue
      cp_pending = false;
      if (it + 1 < my_tiles) copy_v_prepare();  // addresses were worked out in the last softmax block
    };
    // four MFMAs are followed by one copy instruction of the next tile
    auto after4 = [&](int n) {
      if (n < kVCopies) copy_v_issue(n);
      __builtin_amdgcn_sched_barrier(0);
    };

    if (my_tiles > 0) {
      // first tile: nothing to multiply by V yet
      open_mfma_block(0);
      if constexpr (kFp8) {
        s_fp8(0);
#pragma unroll
        for (int n = 0; n < 8; ++n) after4(n);
      } else {
        x8 k_lo[2][4], k_hi[2][4];
        read_k(0, 0, k_lo);
        read_k(0, 4, k_hi);
        __builtin_amdgcn_sched_barrier(0);
        s_math(0, k_lo, 0);
        after4(0);
        after4(1);
        s_math(0, k_lo, 2);
        after4(2);
        after4(3);
        s_math(4, k_hi, 0);
        after4(4);
        after4(5);
        s_math(4, k_hi, 2);
        after4(6);
        after4(7);
      }
      valu_block(0, true);
      for (int it = 1; it < my_tiles; ++it) {
        open_mfma_block(it);
        if constexpr (kFp8) {
          pv_math(0);
          after4(0);
          pv_math(1);
          after4(1);
          pv_math(2);
          after4(2);
          pv_math(3);
          after4(3);
          s_fp8(it);
        } else {
          // K operands are fetched under the MFMAs, half of them at a time, into the registers that
          // the V^T operands free
          x8 k_lo[2][4], k_hi[2][4];
          pv_math(0);
          after4(0);
          pv_math(1);
          after4(1);
          read_k(it, 0, k_lo);
          __builtin_amdgcn_sched_barrier(0);
          pv_math(2);
          after4(2);
          pv_math(3);
          after4(3);
          read_k(it, 4, k_hi);
          __builtin_amdgcn_sched_barrier(0);
          s_math(0, k_lo, 0);
          after4(4);
          s_math(0, k_lo, 2);
          after4(5);
          s_math(4, k_hi, 0);
          after4(6);
          s_math(4, k_hi, 2);
          after4(7);
        }
        valu_block(it, false);
      }
      // last MFMA block: P.V of the last tile
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_s_setprio(3);
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) pv_math(kk);
      __builtin_amdgcn_s_setprio(0);
    } else {
      __builtin_amdgcn_s_barrier();
    }
    for (int i = calls_mine; i < calls_all; ++i) __builtin_amdgcn_s_barrier();
    if (my_tiles == 0) m_run = kNegInf;  // nothing seen: weight 0 in the merge
    }  // !kPipe

    // ---- merge the two kv groups through LDS, then write the row ----
    // (this lane's row, worked out again: what the prologue derived from the lane index would have
    // to live through the main loop, i.e. in scratch memory)
    const int lane_m = fresh_lane();
    const int l32_e = lane_m & 31, g_e = lane_m >> 5;
    const bool row_ok_e = qs * 32 + l32_e < q_rows;
    int tok_e, hq_e;
    row_at(row_ok_e ? qs * 32 + l32_e : q_rows - 1, tok_e, hq_e);
    const int64_t q_tok_e = q_begin + tok_e;
    const int my_head_e = head_q0 + hq_e;
    __syncthreads();  // all tile reads done: the tile buffers can be reused
    f32x4* mo = reinterpret_cast<f32x4*>(smem);
    float* md = reinterpret_cast<float*>(smem + kMergeOBytes);
    if constexpr (kGroups == 2) {
      if (kg == 1) {
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            f32x4 t4;
#pragma unroll
            for (int j = 0; j < 4; ++j) t4[j] = o_acc[dt][i4 * 4 + j];
            mo[(qs * 16 + dt * 4 + i4) * 64 + lane_m] = t4;
          }
        md[(qs * 64 + lane_m) * 2 + 0] = m_run;
        md[(qs * 64 + lane_m) * 2 + 1] = d_part;
      }
      __syncthreads();
    }
    if (wv == kFetchWave) fetch_next((row_it + 1) & 1);
    float m_all = 0.f, d_all = 0.f;  // kv group 0: row maximum and row sum over both groups
    // A lane owns one q row and runs of four d: stored from here, a row would leave as 32 scattered
    // 8-byte pieces per instruction (measured: ~12 k cycles per row).  The finished row goes through
    // a padded LDS tile instead and leaves in 16-byte pieces, 16 consecutive lanes per 256-byte row.
    int ln_out = l32_e;
    asm volatile("" : "+v"(ln_out));  // (not hoisted out of the row loop and spilled)
    uint8_t* const out_row = smem + G::kOutOff + (qs * 32 + ln_out) * kOutRowBytes;
    bool store_row = parts == 1;
    if constexpr (kGroups == 1) {
      // one kv group: the accumulators hold the whole row
      const float d_tot = d_part + __shfl_xor(d_part, 32, 64);
      const float inv = __builtin_amdgcn_rcpf(d_tot);
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          x4 out;
#pragma unroll
          for (int j = 0; j < 4; ++j) out[j] = static_cast<T>(o_acc[dt][i4 * 4 + j] * inv);
          *reinterpret_cast<x4*>(out_row + (dt * 32 + i4 * 8 + g_e * 4) * sizeof(T)) = out;
        }
      if (row_ok_e && p.lse && g_e == 0) p.lse[q_tok_e * p.num_heads + my_head_e] = __builtin_amdgcn_logf(d_tot) + m_run;
    }
    if (kGroups == 2 && kg == 0) {
      const float m1 = md[(qs * 64 + lane_m) * 2 + 0], d1 = md[(qs * 64 + lane_m) * 2 + 1];
      const float m = fmaxf(m_run, m1);
      const float a0 = __builtin_amdgcn_exp2f(m_run - m);
      const float a1 = __builtin_amdgcn_exp2f(m1 - m);
      const float d_lane = d_part * a0 + d1 * a1;
      const float d_tot = d_lane + __shfl_xor(d_lane, 32, 64);
      if (parts == 1) {
        const float inv = __builtin_amdgcn_rcpf(d_tot);
        const float w0 = a0 * inv, w1 = a1 * inv;
        // all sixteen reads of the partner's partial first (the registers of the tile operands are
        // free here), so their latencies overlap
        f32x4 t4[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) t4[e] = mo[(qs * 16 + e) * 64 + lane_m];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            x4 out;
#pragma unroll
            for (int j = 0; j < 4; ++j)
              out[j] = static_cast<T>(o_acc[dt][i4 * 4 + j] * w0 + t4[dt * 4 + i4][j] * w1);
            *reinterpret_cast<x4*>(out_row + (dt * 32 + i4 * 8 + g_e * 4) * sizeof(T)) = out;
          }
        if (row_ok_e && p.lse && g_e == 0)
          p.lse[q_tok_e * p.num_heads + my_head_e] = __builtin_amdgcn_logf(d_tot) + m;
      } else {
        // one part of a row cut at share boundaries: fold kv group 1 in without normalising; the
        // accumulators then hold this workgroup's partial result (reference point m, sum d_tot)
        f32x4 t4[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) t4[e] = mo[(qs * 16 + e) * 64 + lane_m];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int e = 0; e < 16; ++e)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            o_acc[e >> 2][(e & 3) * 4 + j] = o_acc[e >> 2][(e & 3) * 4 + j] * a0 + t4[e][j] * a1;
        m_all = m;
        d_all = d_tot;
      }
    }
    if (kGroups == 2 && parts > 1) {
      // Whoever comes last combines the parts and writes the row.  A workgroup that finds every
      // other part arrived already need not publish its own; otherwise it publishes, then counts
      // itself in, and may still turn out to be the last.
      if (tid == 0)
        s_arrived = __hip_atomic_load(&p.sched[kSchedArrived + split_slot], __ATOMIC_RELAXED,
                                      __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      bool last = s_arrived == parts - 1;
      if (!last) {
        if (kg == 0) {
          // same lane layout as the LDS merge area; two planes of 8-byte pairs, so that each store
          // instruction covers 512 contiguous bytes
          float* part_ws = p.split_ws + static_cast<int64_t>(part_area(split_slot, part)) * kSplitPartFloats;
          const int ln = fresh_lane();
          float* lane_ws = part_ws + (qs * 16 * 2 * 64 + ln) * 2;
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            store_pair_device(lane_ws + e * 256, o_acc[e >> 2][(e & 3) * 4 + 0], o_acc[e >> 2][(e & 3) * 4 + 1]);
            store_pair_device(lane_ws + e * 256 + 128, o_acc[e >> 2][(e & 3) * 4 + 2], o_acc[e >> 2][(e & 3) * 4 + 3]);
          }
          store_pair_device(part_ws + 128 * 128 + (qs * 64 + ln) * 2, m_all, d_all);
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this lane's partial results have left
        __syncthreads();
        if (tid == 0) s_arrived = atomicAdd(&p.sched[kSchedArrived + split_slot], 1);
        __syncthreads();
        last = s_arrived == parts - 1;
      }
      if (last) {
        if (kg == 0) {
          // The parts are added in part order, this workgroup's own from its registers (the same
          // values it would have published), the others read back: the row does not depend on
          // which part came last.
          auto part_base = [&](int i) {
            return p.split_ws + static_cast<int64_t>(part_area(split_slot, i)) * kSplitPartFloats;
          };
          float m_p[kMaxSplitParts], d_p[kMaxSplitParts];
          const float m_own = m_all, d_own = d_all;
          m_all = kNegInf;
          for (int i = 0; i < parts; ++i) {
            if (i == part) {
              m_p[i] = m_own;
              d_p[i] = d_own;
            } else {
              load_pair_device(part_base(i) + 128 * 128 + (qs * 64 + lane_m) * 2, m_p[i], d_p[i]);
            }
            m_all = fmaxf(m_all, m_p[i]);
          }
          d_all = 0.f;
          f32x16 acc[4];
#pragma unroll
          for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[dt][e] = 0.f;
          const int ln = fresh_lane();
          for (int i = 0; i < parts; ++i) {
            const float a = __builtin_amdgcn_exp2f(m_p[i] - m_all);
            d_all = __builtin_fmaf(d_p[i], a, d_all);
            if (i == part) {
#pragma unroll
              for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[dt][e] = __builtin_fmaf(o_acc[dt][e], a, acc[dt][e]);
            } else {
              const float* lane_ws = part_base(i) + (qs * 16 * 2 * 64 + ln) * 2;
              // all loads of the part in flight together
              float u[16][4];
#pragma unroll
              for (int e = 0; e < 16; ++e) {
                load_pair_device(lane_ws + e * 256, u[e][0], u[e][1]);
                load_pair_device(lane_ws + e * 256 + 128, u[e][2], u[e][3]);
              }
              __builtin_amdgcn_sched_barrier(0);
#pragma unroll
              for (int e = 0; e < 16; ++e)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                  acc[e >> 2][(e & 3) * 4 + j] = __builtin_fmaf(u[e][j], a, acc[e >> 2][(e & 3) * 4 + j]);
            }
          }
          const float inv = __builtin_amdgcn_rcpf(d_all);
#pragma unroll
          for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
              x4 out;
#pragma unroll
              for (int j = 0; j < 4; ++j) out[j] = static_cast<T>(acc[dt][i4 * 4 + j] * inv);
              *reinterpret_cast<x4*>(out_row + (dt * 32 + i4 * 8 + g_e * 4) * sizeof(T)) = out;
            }
          if (row_ok_e && p.lse && g_e == 0)
            p.lse[q_tok_e * p.num_heads + my_head_e] = __builtin_amdgcn_logf(d_all) + m_all;
        }
        if (tid == 0) p.sched[kSchedArrived + split_slot] = 0;  // re-armed for the next launch
        store_row = true;
      }
      // (nothing may be in flight into registers where this path joins the one that stores a row:
      // the compiler would wait there for everything, the row's stores included)
      __builtin_amdgcn_s_waitcnt(0x0f70);
    }
    if (store_row && kg == 0) {
      // A wavefront stores the 32 rows it has just written to the LDS tile itself: no barrier, so
      // the other kv group (whose first wavefront is fetching the next row's record meanwhile) is not
      // waited for here but at the top of the next row.
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wavefront's rows are in the tile
      T* dst = op + static_cast<int64_t>(q_begin) * p.o_sn + static_cast<int64_t>(head_q0) * p.o_sh;
      // (the lane index is worked out afresh here: otherwise the per-lane address terms are computed once
      // per kernel, spilled, and every reload waits for the store before it)
      const int ln = fresh_lane();
      const int r0 = qs * 32 + (ln >> 4), chunk = ln & 15;
      u32x4 v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i)
        v[i] = *reinterpret_cast<const u32x4*>(smem + G::kOutOff + (r0 + i * 4) * kOutRowBytes + chunk * 16);
      T* d0 = dst + chunk * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        // (streaming stores: O is not read again here and should not push K and V out of the L2;
        // 3 MB less fetched per FLUX-sized launch at the same speed.  The same hint on the Q copies
        // takes another 6 MB off and 0.6 % of speed: not used.)
        if (r0 + i * 4 < q_rows) __builtin_nontemporal_store(v[i], reinterpret_cast<u32x4*>(d0 + row_off(r0 + i * 4, p.o_sn, p.o_sh)));
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

template <typename T, bool kFp8, bool kQLo, bool kKLo, int kGroups = 2, bool kPipe = false, bool kGqaPack = false,
          bool kCap = false>
int launch(const FaParams& p, int64_t max_rows, hipStream_t stream) {
  constexpr int kSmemBytes = Geom<kFp8, kKLo, kGroups>::kSmemBytes;
  // (the attribute belongs to the kernel's code object on one device: set once per device; the flags
  // are atomic because host threads may launch concurrently, and setting it twice is harmless)
  static std::atomic<bool> attr_set[64] = {};
  int dev = 0;
  FO_HIP_CALL(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64 || !attr_set[dev].load(std::memory_order_acquire)) {
    FO_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(&sparse_fa_kernel<T, kFp8, kQLo, kKLo, kGroups, kPipe, kGqaPack, kCap>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kSmemBytes));
    if (dev >= 0 && dev < 64) attr_set[dev].store(true, std::memory_order_release);
  }
  int num_cu = fo_num_cu();
  if (num_cu <= 0) return fo::fail(FO_ERR_HIP, "sparse_fa: no device");
  int64_t grid = num_cu * (3 - kGroups);  // persistent workgroups: one per CU, or two of one kv group each (LDS bound)
  // (with even shares every workgroup may hold a part of a row; otherwise at most one row each)
  if (!(p.split_ws && p.shares) && grid > max_rows) grid = max_rows;
  sparse_fa_kernel<T, kFp8, kQLo, kKLo, kGroups, kPipe, kGqaPack, kCap><<<static_cast<unsigned>(grid), kGroups * kGroupThreads, kSmemBytes, stream>>>(p);
  FO_CHECK_LAUNCH();
  return FO_OK;
}

}  // namespace

namespace {
std::atomic<int> g_variant{0};
}

extern "C" int fo_sparse_fa_set_variant(int variant) {
  FO_REQUIRE(variant >= 0 && variant <= 2, "sparse_fa: variant must be 0 (automatic), 1 or 2");
  g_variant.store(variant, std::memory_order_relaxed);
  return FO_OK;
}

extern "C" int64_t fo_sparse_fa_split_workspace_bytes(void) {
  // two areas per share, one share per workgroup = per CU
  return static_cast<int64_t>(2) * fo_num_cu() * kSplitPartFloats * sizeof(float);
}

extern "C" int fo_sparse_fa_run(const void* q, const void* k, const void* v, void* o, float* lse,
                                int dtype, const void* q_lo, const void* k_lo, const float* q_scale,
                                const float* k_scale,
                                int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n,
                                int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h,
                                int64_t o_stride_n, int64_t o_stride_h, const int32_t* qo_indptr,
                                const int32_t* kv_indptr, const int32_t* q_blk_base,
                                const int32_t* kv_blk_base, int32_t n_q_blocks,
                                int32_t n_kv_blocks, const int32_t* row_req,
                                const int32_t* row_qb, const int32_t* row_head,
                                const int32_t* kv_row_ptr, const int32_t* kv_idx,
                                const int32_t* order, int32_t* sched, int64_t max_rows,
                                int32_t num_heads, int32_t num_kv_heads, int32_t gqa_packed, int32_t head_dim,
                                int32_t block_q, int32_t block_kv, float sm_scale, float logits_soft_cap,
                                const int32_t* shares, void* split_workspace, int64_t split_workspace_bytes,
                                void* stream) {
  FO_REQUIRE(head_dim == kHeadDim, "sparse_fa: head_dim %d is not supported (only 128)", head_dim);
  FO_REQUIRE(block_q == kBlockQ && block_kv == kBlockKV,
             "sparse_fa: sparse block sizes (%d, %d) are not supported (only 128, 128)", block_q,
             block_kv);
  FO_REQUIRE(dtype == FO_BF16 || dtype == FO_F16 || dtype == FO_FP8_E4M3,
             "sparse_fa: unsupported dtype code %d", dtype);
  FO_REQUIRE(num_heads > 0 && max_rows >= 0, "sparse_fa: bad sizes");
  FO_REQUIRE(num_kv_heads > 0 && num_heads % num_kv_heads == 0,
             "sparse_fa: num_qo_heads %d is not a multiple of num_kv_heads %d", num_heads, num_kv_heads);
  FO_REQUIRE(gqa_packed == 0 || gqa_packed == 1, "sparse_fa: gqa_packed must be 0 or 1");
  FO_REQUIRE(logits_soft_cap >= 0.f && logits_soft_cap < __builtin_inff(),
             "sparse_fa: logits_soft_cap must be a finite value >= 0 (0: no cap)");
  FO_REQUIRE(logits_soft_cap == 0.f || dtype != FO_FP8_E4M3, "sparse_fa: the logits soft cap is not built for fp8 q/k");
  FO_REQUIRE(!gqa_packed || dtype != FO_FP8_E4M3,
             "sparse_fa: fp8 q (one scale per q head and token block) is not built for packed tiles of "
             "several q heads");
  if (max_rows == 0) return FO_OK;
  FO_REQUIRE(q && k && v && o && qo_indptr && kv_indptr && row_req && row_qb && row_head &&
                 kv_row_ptr && kv_idx && order && sched,
             "sparse_fa: null pointer");
  const int64_t strides[8] = {q_stride_n, q_stride_h, k_stride_n, k_stride_h,
                              v_stride_n, v_stride_h, o_stride_n, o_stride_h};
  for (int i = 0; i < 8; ++i)
    FO_REQUIRE(strides[i] % (dtype == FO_FP8_E4M3 && i < 4 ? 16 : 8) == 0 && strides[i] > 0,
               "sparse_fa: strides must be positive multiples of 16 bytes (128-bit accesses)");
  FO_REQUIRE(q_stride_n < (int64_t(1) << 23) && k_stride_n < (int64_t(1) << 23) &&
                 v_stride_n < (int64_t(1) << 23),
             "sparse_fa: q/k/v token strides must be below 2^23 elements (32-bit tile offsets)");
  if (dtype == FO_FP8_E4M3)
    FO_REQUIRE(q_scale && k_scale && q_blk_base && kv_blk_base && n_q_blocks > 0 && n_kv_blocks > 0,
               "sparse_fa: fp8 q/k need q_scale, k_scale, the block numbering and the scale row lengths");
  FO_REQUIRE(q_lo == nullptr || dtype == FO_FP8_E4M3, "sparse_fa: q_lo is the second term of an fp8 q");
  FO_REQUIRE(k_lo == nullptr || q_lo != nullptr, "sparse_fa: k_lo (second term of an fp8 k) needs q_lo as well");
  for (const void* ptr : {q, k, v, static_cast<const void*>(o), q_lo, k_lo})
    FO_REQUIRE((reinterpret_cast<uintptr_t>(ptr) & 15) == 0,
               "sparse_fa: q/k/v/o must be 16-byte aligned");

  FaParams p;
  p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse;
  p.q_lo = q_lo; p.k_lo = k_lo; p.q_scale = q_scale; p.k_scale = k_scale;
  p.q_sn = q_stride_n; p.q_sh = q_stride_h; p.k_sn = k_stride_n; p.k_sh = k_stride_h;
  p.v_sn = v_stride_n; p.v_sh = v_stride_h; p.o_sn = o_stride_n; p.o_sh = o_stride_h;
  p.qo_indptr = qo_indptr; p.kv_indptr = kv_indptr;
  p.q_blk_base = q_blk_base; p.kv_blk_base = kv_blk_base;
  p.row_req = row_req; p.row_qb = row_qb; p.row_head = row_head;
  p.kv_row_ptr = kv_row_ptr; p.kv_idx = kv_idx; p.order = order; p.sched = sched;
  // even shares need both the decoder's share table and room for partial results (without them
  // the rows are taken whole from the queues, which the decoder fills either way)
  p.split_ws = nullptr;
  p.shares = nullptr;
  if (shares != nullptr) {
    FO_REQUIRE(split_workspace != nullptr && split_workspace_bytes >= fo_sparse_fa_split_workspace_bytes(),
               "sparse_fa: the work list was decoded for even shares, which need a split workspace of "
               "fo_sparse_fa_split_workspace_bytes() bytes");
    FO_REQUIRE((reinterpret_cast<uintptr_t>(split_workspace) & 15) == 0,
               "sparse_fa: split_workspace must be 16-byte aligned");
    p.split_ws = static_cast<float*>(split_workspace);
    p.shares = shares;
  }
  p.num_heads = num_heads;
  // packed tiles: row_head is the kv head already, and a tile's rows spread over its q heads
  const bool packed = gqa_packed && num_heads != num_kv_heads;
  p.kv_group = packed ? 1 : num_heads / num_kv_heads;
  p.gqa_pack = packed ? num_heads / num_kv_heads : 0; p.n_q_blocks = n_q_blocks; p.n_kv_blocks = n_kv_blocks;
  p.sm_scale_log2 = sm_scale * 1.44269504088896340736f;
  p.cap_log2 = 0.f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (logits_soft_cap > 0.f) {
    // (reference: soft_cap_pre_tanh_scale = sm_scale / cap, sm_scale_log2 = log2(e) * cap, variants.cuh:43-56)
    p.cap_log2 = logits_soft_cap * 1.44269504088896340736f;
    p.sm_scale_log2 = 2.f * 1.44269504088896340736f * sm_scale / logits_soft_cap;
    if (p.gqa_pack)
      return dtype == FO_BF16 ? launch<__bf16, false, false, false, 2, false, true, true>(p, max_rows, s)
                              : launch<_Float16, false, false, false, 2, false, true, true>(p, max_rows, s);
    return dtype == FO_BF16 ? launch<__bf16, false, false, false, 2, false, false, true>(p, max_rows, s)
                            : launch<_Float16, false, false, false, 2, false, false, true>(p, max_rows, s);
  }
  // Long lists (many rows per CU) run as two independent 4-wavefront workgroups per CU with the
  // software-pipelined loop; short ones as one 8-wavefront workgroup whose two kv groups share a row
  // (half the latency per row, and rows can be cut into even shares).  The list's length lives on the
  // device: the choice is made from its upper bound max_rows, unless fo_sparse_fa_set_variant() fixed
  // it.  The one-group form needs 16-bit operands, at most 3072 kv blocks per request and kv spans
  // below 4 GiB (32-bit copy offsets): n_kv_blocks, the batch's total, bounds both.
  const int64_t span = static_cast<int64_t>(n_kv_blocks) * kBlockKV * 2;
  const bool one_group_ok = (dtype == FO_BF16 || dtype == FO_F16) && n_kv_blocks > 0 &&
                            n_kv_blocks <= kMaxRowBlocksOneGroup && span * k_stride_n < (int64_t(1) << 32) &&
                            span * v_stride_n < (int64_t(1) << 32);
  const int variant = g_variant.load(std::memory_order_relaxed);
  const bool one_group = one_group_ok && (variant == 1 || (variant == 0 && max_rows >= static_cast<int64_t>(8) * fo_num_cu()));
  if (p.gqa_pack) {  // packed tiles of several q heads: the row mapping is compiled in
    if (dtype == FO_BF16)
      return one_group ? launch<__bf16, false, false, false, 1, true, true>(p, max_rows, s)
                       : launch<__bf16, false, false, false, 2, false, true>(p, max_rows, s);
    return one_group ? launch<_Float16, false, false, false, 1, true, true>(p, max_rows, s)
                     : launch<_Float16, false, false, false, 2, false, true>(p, max_rows, s);
  }
  if (dtype == FO_BF16)
    return one_group ? launch<__bf16, false, false, false, 1, true>(p, max_rows, s)
                     : launch<__bf16, false, false, false, 2>(p, max_rows, s);
  if (dtype == FO_F16)
    return one_group ? launch<_Float16, false, false, false, 1, true>(p, max_rows, s)
                     : launch<_Float16, false, false, false, 2>(p, max_rows, s);
  if (k_lo != nullptr) return launch<__bf16, true, true, true>(p, max_rows, s);
  if (q_lo != nullptr) return launch<__bf16, true, true, false>(p, max_rows, s);
  return launch<__bf16, true, false, false>(p, max_rows, s);
}
