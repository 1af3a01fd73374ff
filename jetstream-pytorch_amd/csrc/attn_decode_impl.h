// Streaming GQA decode attention kernel for gfx950, head_dim 128 (template
// body; attn_decode_i8.hip and attn_decode_bf16.hip instantiate it).
//
// One workgroup per compute unit holds kGroups independent groups of
// wavefronts; a group walks its share of the planned (chunk, KV head) items as
// one stream of 32-position tiles:
//
//   producer wave   copies each tile's K rows, V rows and per-position scales
//                   from HBM straight into the group's LDS ring with
//                   direct-to-LDS loads (no registers), several tiles ahead
//                   and regardless of item boundaries, and each item's query
//                   rows ahead of its first tile.  HBM sees full 1 KiB bursts of
//                   contiguous cache rows; a first touch of a new cache row
//                   (several microseconds with its TLB miss) is hidden behind
//                   the tiles already in the ring.
//   consumer waves  take tiles round-robin out of the ring, turn int8 codes
//                   into float16 operands with byte permutes (exact; bf16
//                   caches go in as they are) and run
//                       S^T = K . Q^T   v_mfma_f32_16x16x32_f16 / _bf16,
//                                       positions on M, the rep*q_rows query
//                                       rows on N
//                       O^T = V^T . P^T positions on the contraction index
//                   with an online softmax in between.  The score
//                   accumulators of lane (row r, group g) are exactly the
//                   probabilities that lane feeds to the second MFMA, so
//                   probabilities never cross lanes.
//
// A consumer wave is bound by latencies, not by issue slots, so the kernel
// wants many of them per SIMD; several groups in one workgroup (instead of
// several workgroups per unit) make the wave placement over the SIMDs even.
// Waves never meet at a workgroup barrier after set-up: ring slots are handed
// over through LDS counters, and the consumer that delivers the last part of an
// item folds the parts and writes the slot's output (one chunk) or parks the
// chunk's float32 partial in memory and counts the chunk as arrived (several
// chunks; a merge item at the end of some worker's sequence folds those, see
// merge_item).  Every wait
// is bounded: a wave that waits too long raises an abort flag, every wave of
// the workgroup leaves, and a sticky word in the workspace's state block tells
// the host that the launch's results are not to be used (jpt_attn_status), so
// a logic error shows up as an error, never as a hung GPU.
#pragma once

#include <math.h>

#include <type_traits>

#include "attn_common.h"
#include "attn_plan.h"

// Development aid, off in the product library: with JPT_ATTN_TIMELINE defined every wave of
// the first 256 workgroups leaves four words in the workspace's state block (from byte 1024:
// [workgroup][group][producer, consumers 0..2][start, first tile, end, tiles | items << 16],
// times on the constant 100 MHz clock), from which attn_timeline.py derives when workers
// start, stream and end.  build_lib.py --timeline builds that library beside the product's.
#ifdef JPT_ATTN_TIMELINE
#define JPT_TL(...) __VA_ARGS__
#else
#define JPT_TL(...)
#endif

namespace jpt {
namespace decode {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef const __attribute__((address_space(1))) void* global_ptr;
typedef __attribute__((address_space(3))) void* lds_ptr;

constexpr int kConsumers = 3;
constexpr int kGroups = 2;
constexpr int kWavesPerSimd = 2;
constexpr int kGroupWaves = kConsumers + 1;  // wave 0 of a group is its producer
constexpr int kWaves = kGroups * kGroupWaves;
constexpr int kThreads = kWaves * 64;
constexpr int kSideBytes = 512;     // ks | vs | mask, 128 bytes each at most
constexpr int kOStride = 140;       // padded LDS row of 128 outputs
constexpr int kLdsBudget = 160 * 1024 / kGroups - 512;  // per group; one workgroup per compute unit
constexpr int kSpinLimit = 1 << 18;  // tens of milliseconds
constexpr int kMergeSpinLimit = 1 << 16;  // polls of a merge's wait for other workgroups' chunks
// Cache policy of the loads that stream the cache (keys, values, their scales):
// non-temporal - every byte is read once per launch, and lines kept for it in
// the caches only push out what is read again (query rows, page ids, masks).
// Measured on the same tensors: all slots at 8192 positions 5.5 -> 6.2 TB/s.
constexpr int kStreamOnce = 2;  // the NT bit of the instruction's cache-policy field
constexpr int kListedItems = 64;     // a worker's first items, read into LDS at start
constexpr int kStagedPages = 64;     // page ids of an item kept in LDS (later pages are read one by one)
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// 2^x by the hardware instruction alone.  Arguments here are <= 0 (or -inf);
// results below the normal range flush to zero, which is right for them.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// column d = 32g + c of an output row lives at 36g + c: the column groups of a
// wave's writers fall on different banks and runs of eight stay 16-byte aligned
__device__ __forceinline__ int o_col(int d) { return d + 4 * (d >> 5); }

enum ScaleKind { kNoScale = 0, kScaleF32 = 1, kScaleBF16 = 2 };

template <typename KV, int SCALE, bool MASK, int RC>
struct Config {
  static constexpr int kElem = sizeof(KV);
  static constexpr int kRowBytes = kD * kElem;
  static constexpr int kTileBytes = kTile * kRowBytes;            // K or V of one tile
  static constexpr int kSlotBytes = 2 * kTileBytes + kSideBytes;
  static constexpr int kLoadsPerTile = 2 * kTileBytes / 1024 + (SCALE ? 1 : 0) + (MASK ? 1 : 0);
  // query rows of the next items, staged by the producer
  static constexpr int kQBufs = RC <= 8 ? 4 : 2;
  static constexpr int kQBytes = kQBufs * RC * kD * 2;
  static constexpr int kQLoadsMax = (RC + 3) / 4;  // 1 KiB (four rows) a load
  static constexpr int kFoldPart = kConsumers * RC * (kOStride + 2) * 4;
  // ring slots: every one may hold a tile in flight, and the wave's load
  // counter counts to 63 (the producer checks the room before each issue)
  static constexpr int kSlotsByCount = 63 / kLoadsPerTile;
  static constexpr int kSlotsWith2 = (kLdsBudget - kQBytes - 2 * kFoldPart) / kSlotBytes;
  static constexpr int kEnough = kSlotsByCount < 5 ? kSlotsByCount : 5;
  static constexpr int kFoldBufs = kSlotsWith2 >= kEnough ? 2 : 1;
  static constexpr int kSlotsByLds = (kLdsBudget - kQBytes - kFoldBufs * kFoldPart) / kSlotBytes;
  static constexpr int kSlots = kSlotsByLds < kSlotsByCount ? kSlotsByLds : kSlotsByCount;
  static_assert(kSlots >= 2, "LDS ring too small");
};

// LDS word access the compiler does not see as LDS traffic.  The producer
// wave keeps direct-to-LDS loads in flight all the time; the compiler orders
// every LDS access it knows of after ALL of them (it cannot tell the ring from
// the counters), which would drain the pipeline at each hand-over.
typedef __attribute__((address_space(3))) int* lds_int_ptr;
__device__ __forceinline__ int lds_peek(const int* p) {
  const uint32_t addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_int_ptr)p));
  int v;
  asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
  return v;
}
typedef __attribute__((ext_vector_type(4))) int i32x4;
__device__ __forceinline__ i32x4 lds_peek4(const int* p) {
  const uint32_t addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_int_ptr)p));
  i32x4 v;
  asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
  return v;
}
__device__ __forceinline__ void lds_poke(int* p, int v) {
  const uint32_t addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_int_ptr)p));
  asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(v) : "memory");
}

__device__ __forceinline__ void lds_poke4(void* p, i32x4 v) {
  const uint32_t addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_int_ptr)p));
  asm volatile("ds_write_b128 %0, %1" : : "v"(addr), "v"(v) : "memory");
}
typedef __attribute__((ext_vector_type(2))) int i32x2;
__device__ __forceinline__ void lds_poke2(void* p, i32x2 v) {
  const uint32_t addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_int_ptr)p));
  asm volatile("ds_write_b64 %0, %1" : : "v"(addr), "v"(v) : "memory");
}

// An LDS word every lane reads alike, as a wave-uniform (scalar) value: what
// the producer branches on stays out of the vector condition path.
__device__ __forceinline__ int lds_peek_uniform(const int* p) {
  return __builtin_amdgcn_readfirstlane(lds_peek(p));
}

// Load through the scalar data path.  `p` must be the same in every lane and
// must not be written while the kernel runs (plan entries and page tables are
// written by earlier work on the stream).  Keeps such loads out of the vector
// memory counter, which the producer wave reserves for its tile loads.
template <typename T>
__device__ __forceinline__ T load_uniform(const T* p) {
  typedef const __attribute__((address_space(4))) T* constant_ptr;
  return *(constant_ptr)p;
}

// Maximum over the wave's 64 lanes, the same value in every lane.  Data-parallel
// primitives inside the 16-lane rows (quad swaps, then the row's halves and the
// row mirrored), four lane reads across the rows: no LDS round trips.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float row_max(float v) {
  v = fmaxf(v, dpp_move<0xB1>(v));   // quad_perm [1, 0, 3, 2]
  v = fmaxf(v, dpp_move<0x4E>(v));   // quad_perm [2, 3, 0, 1]
  v = fmaxf(v, dpp_move<0x141>(v));  // row_half_mirror
  v = fmaxf(v, dpp_move<0x140>(v));  // row_mirror
  return v;
}
__device__ __forceinline__ float row_sum(float v) {  // over the 16 lanes of a row, in every lane of it
  v += dpp_move<0xB1>(v);
  v += dpp_move<0x4E>(v);
  v += dpp_move<0x141>(v);
  v += dpp_move<0x140>(v);
  return v;
}
__device__ __forceinline__ float rows_max(float r) {
  const int bits = __builtin_bit_cast(int, r);
  const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0));
  const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16));
  const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32));
  const float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48));
  return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// Combines a value over the four 16-lane rows of the wave (lanes r, 16 + r,
// 32 + r, 48 + r end up with the same result) with the row-swap instructions
// of gfx950: v_permlane16_swap exchanges rows 1 and 3 of one operand with rows
// 0 and 2 of the other, v_permlane32_swap the upper half of one with the lower
// half of the other, so two swaps and two combines do it in the vector ALU,
// with no trip through the LDS crossbar.  The second operand is a copy the
// optimiser cannot see through (the swap of a register with itself is not
// what the instruction does).
template <typename F>
__device__ __forceinline__ float across_rows(float v, F combine) {
  int a = __builtin_bit_cast(int, v), c = a;
  asm volatile("" : "+v"(c));
  const auto s16 = __builtin_amdgcn_permlane16_swap(a, c, false, false);
  const int lo16 = s16[0], hi16 = s16[1];  // named: a bit cast straight from the element reads element 0 twice
  v = combine(__builtin_bit_cast(float, lo16), __builtin_bit_cast(float, hi16));
  a = __builtin_bit_cast(int, v);
  c = a;
  asm volatile("" : "+v"(c));
  const auto s32 = __builtin_amdgcn_permlane32_swap(a, c, false, false);
  const int lo32 = s32[0], hi32 = s32[1];
  return combine(__builtin_bit_cast(float, lo32), __builtin_bit_cast(float, hi32));
}
__device__ __forceinline__ float max_across_rows(float v) {
  return across_rows(v, [](float x, float y) { return fmaxf(x, y); });
}
__device__ __forceinline__ float sum_across_rows(float v) {
  return across_rows(v, [](float x, float y) { return x + y; });
}

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding)
constexpr int vmcnt_imm(int n) { return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14); }

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  bf16x2 t = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
  return __builtin_bit_cast(uint32_t, t);
}
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  f16x2 t = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
  return __builtin_bit_cast(uint32_t, t);
}
template <typename Op>
__device__ __forceinline__ Op as_op(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  uint4 u = make_uint4(a, b, c, d);
  return __builtin_bit_cast(Op, u);
}

// One tile in a consumer's registers.  Lane (r, g) holds elements [32g, 32g+32)
// of positions r and 16+r (K) and elements [8r, 8r+8) of its eight probability
// positions (V).  In LDS a row is stored as 16-byte pieces, piece p of
// position t at piece slot p ^ (t & 7) (int8) or p ^ (t & 15) (bf16), which
// spreads both access patterns over the banks.
template <typename KV>
struct Tile;

// int8 codes enter the matrix cores as float16 without a conversion
// instruction: with the sign bit flipped a code byte is u = code + 128, and
// the halfword 0x6400 | u is the float16 number 1024 + u = code + 1152
// exactly.  A byte permute builds two such halfwords at once.  The constant
// 1152 is taken out again where it is a rank-one term: 1152 * sum(q) is the
// same for every position of a query row (the score accumulators start from
// its negative), and 1152 * sum(weights) per row is accumulated by one more
// MFMA against a tile of ones and subtracted when the item is finished.
template <>
struct Tile<int8_t> {
  typedef f16x8 Op;
  static constexpr float kBias = 1152.f;
  uint4 ka[2], kb[2];
  uint2 v[8];
  __device__ __forceinline__ void read(const char* ks, const char* vs, int r, int g, const int* pos) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int t = r + 16 * half;
      const uint4* row = reinterpret_cast<const uint4*>(ks + t * 128);
      uint4 x = row[(2 * g) ^ (t & 7)], y = row[(2 * g + 1) ^ (t & 7)];
      x.x ^= 0x80808080u; x.y ^= 0x80808080u; x.z ^= 0x80808080u; x.w ^= 0x80808080u;
      y.x ^= 0x80808080u; y.y ^= 0x80808080u; y.z ^= 0x80808080u; y.w ^= 0x80808080u;
      if (half == 0) { ka[0] = x; ka[1] = y; } else { kb[0] = x; kb[1] = y; }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int t = pos[i];
      v[i] = *reinterpret_cast<const uint2*>(vs + t * 128 + 16 * ((r >> 1) ^ (t & 7)) + 8 * (r & 1));
    }
  }
  // bytes (b0, b1) or (b2, b3) of w as two float16 1024 + b
  __device__ __forceinline__ static uint32_t widen(uint32_t w, bool upper) {
    return __builtin_amdgcn_perm(0x64646464u, w, upper ? 0x04030402u : 0x04010400u);
  }
  __device__ __forceinline__ Op k_op(bool second, int kk) const {
    const uint4& q = second ? kb[kk >> 1] : ka[kk >> 1];
    const uint32_t w0 = (kk & 1) ? q.z : q.x, w1 = (kk & 1) ? q.w : q.y;
    return as_op<Op>(widen(w0, false), widen(w0, true), widen(w1, false), widen(w1, true));
  }
  // byte j of positions 2i and 2i+1, sign bits flipped and the exponent set in one xor
  __device__ __forceinline__ uint32_t v_pair(int i, int j) const {
    const uint32_t lo = j < 4 ? v[2 * i].x : v[2 * i].y, hi = j < 4 ? v[2 * i + 1].x : v[2 * i + 1].y;
    const uint32_t sel = 0x0c000c00u | static_cast<uint32_t>(j & 3) | (static_cast<uint32_t>(4 + (j & 3)) << 16);
    return __builtin_amdgcn_perm(hi, lo, sel) ^ 0x64806480u;
  }
  __device__ __forceinline__ Op v_op(int j) const {
    return as_op<Op>(v_pair(0, j), v_pair(1, j), v_pair(2, j), v_pair(3, j));
  }
  __device__ __forceinline__ static f32x4 mfma(Op a, Op b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  __device__ __forceinline__ static uint32_t pack(float lo, float hi) { return pack_f16(lo, hi); }
  __device__ __forceinline__ static Op ones() {
    return as_op<Op>(0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u);
  }
};

template <>
struct Tile<__bf16> {
  typedef bf16x8 Op;
  static constexpr float kBias = 0.f;
  uint4 ka[4], kb[4];
  uint4 v[8];
  __device__ __forceinline__ void read(const char* ks, const char* vs, int r, int g, const int* pos) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int t = r + 16 * half;
      const uint4* row = reinterpret_cast<const uint4*>(ks + t * 256);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint4 x = row[(4 * g + i) ^ (t & 15)];
        if (half == 0) ka[i] = x; else kb[i] = x;
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int t = pos[i];
      v[i] = *reinterpret_cast<const uint4*>(vs + t * 256 + 16 * (r ^ (t & 15)));
    }
  }
  __device__ __forceinline__ Op k_op(bool second, int kk) const {
    return __builtin_bit_cast(Op, second ? kb[kk] : ka[kk]);
  }
  __device__ __forceinline__ uint32_t v_word(int i, int j) const {
    const int w = j >> 1;
    return w == 0 ? v[i].x : w == 1 ? v[i].y : w == 2 ? v[i].z : v[i].w;
  }
  __device__ __forceinline__ Op v_op(int j) const {
    const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
    return as_op<Op>(__builtin_amdgcn_perm(v_word(1, j), v_word(0, j), sel),
                     __builtin_amdgcn_perm(v_word(3, j), v_word(2, j), sel),
                     __builtin_amdgcn_perm(v_word(5, j), v_word(4, j), sel),
                     __builtin_amdgcn_perm(v_word(7, j), v_word(6, j), sel));
  }
  __device__ __forceinline__ static f32x4 mfma(Op a, Op b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  __device__ __forceinline__ static uint32_t pack(float lo, float hi) { return pack_bf16(lo, hi); }
  __device__ __forceinline__ static Op ones() { return as_op<Op>(0, 0, 0, 0); }  // unused
};


// One work item: a chunk of one slot for one KV head.
struct Item {
  int slot, start, count, part, n_chunks, h;
  int len;  // positions of the whole slot
  bool valid;
  // folds the partials of a split slot (part = its first partial record) instead of attending positions
  __device__ __forceinline__ bool merge() const { return start < 0; }
};

// NEW: how the step's new token comes (kNew*): compile-time, because each of these few
// branches in the producer's and the consumers' loops costs scalar registers and code the
// common launch never runs (the headline workload's launch 33.05 -> 32.5 us on the same
// tensors when they became constants).
template <typename KV, bool PAGED, int SCALE, bool MASK, int RC, int NEW>
__global__ void __launch_bounds__(kThreads, kWavesPerSimd) attn_decode_kernel(FastParams p) {
  using C = Config<KV, SCALE, MASK, RC>;
  const jpt_attn_args& a = p.a;
  // The kernel's arguments span several cache lines, which the compiler would
  // fetch one after another as the code first needs them, a trip to memory
  // each.  One word of every line is asked for here, all at once.
  {
    typedef const __attribute__((address_space(4))) int* const_int_ptr;
    const_int_ptr args = (const_int_ptr)__builtin_amdgcn_kernarg_segment_ptr();
    int touched = 0;
#pragma unroll
    for (unsigned at = 0; at < sizeof(FastParams); at += 64) touched += args[at / 4];
    asm volatile("" : : "s"(touched));
  }
  __shared__ __attribute__((aligned(1024))) char ring_all[kGroups][C::kSlots * C::kSlotBytes];
  __shared__ __attribute__((aligned(16))) float sm_o_all[kGroups][C::kFoldBufs][kConsumers][RC][kOStride];
  __shared__ __attribute__((aligned(16))) uint16_t sm_q_all[kGroups][C::kQBufs][RC][kD];
  // per query row, written by the producer with the row's float16 operand (int8 codes only):
  // the power of two taken out of the row, and minus the bias term of its scores
  __shared__ __attribute__((aligned(8))) float sm_qmeta_all[kGroups][C::kQBufs][RC][2];
  __shared__ float sm_m_all[kGroups][C::kFoldBufs][kConsumers][RC];
  __shared__ float sm_l_all[kGroups][C::kFoldBufs][kConsumers][RC];
  __shared__ int sm_filled_all[kGroups][C::kSlots];   // times the producer filled this slot
  __shared__ int sm_freed_all[kGroups][C::kSlots];    // times a consumer emptied it
  __shared__ int sm_qtaken_all[kGroups][C::kQBufs];   // consumers that took this query buffer
  __shared__ int sm_arrived_all[kGroups][C::kFoldBufs];
  __shared__ int sm_folded_all[kGroups][C::kFoldBufs];
  __shared__ int sm_pair_ready[C::kFoldBufs];  // items whose parts group 1 has left for group 0 to fold (paired chunks)
  __shared__ int sm_abort;
  __shared__ __attribute__((aligned(16))) int sm_items_all[kGroups][kListedItems][8];
  // page ids of the item being issued and of the next one (paged caches)
  __shared__ int sm_pages_all[PAGED ? kGroups : 1][2][kStagedPages];

  const int tid = threadIdx.x, lane = tid & 63;
  const int hw_wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, and known to be
  // Waves of a workgroup go round the four SIMDs in order.  Waves 0 and 1 are
  // the producers, which mostly sleep; waves 4 and 5, on the same SIMDs, are
  // each group's consumer 0, which has its SIMD nearly to itself; consumers 1
  // and 2 of both groups share SIMDs 2 and 3 in pairs.  (With both producers
  // on one SIMD and the six consumers on the other three, long slots ran 5 %
  // slower.)
  static_assert(kGroups == 2 && kConsumers == 3, "the role table below is for two groups of 1 + 3 waves");
  const int group = static_cast<int>((0xE2u >> hw_wave) & 1u);                  // 0 1 0 0 0 1 1 1
  // role index: consumers 0..kConsumers-1, producer kConsumers
  const int wave = static_cast<int>((0x909Fu >> (2 * hw_wave)) & 3u);           // 3 3 1 2 0 0 1 2
  for (int i = tid; i < kGroups * C::kSlots; i += kThreads) {
    (&sm_filled_all[0][0])[i] = 0;
    (&sm_freed_all[0][0])[i] = 0;
  }
  if (tid < kGroups * C::kFoldBufs) {
    (&sm_arrived_all[0][0])[tid] = 0;
    (&sm_folded_all[0][0])[tid] = 0;
    if (tid < C::kFoldBufs) sm_pair_ready[tid] = 0;
  }
  if (tid < kGroups * C::kQBufs) (&sm_qtaken_all[0][0])[tid] = 0;

  if (tid == 0) sm_abort = 0;
  JPT_TL(
  int* const tl_rec = reinterpret_cast<int*>(reinterpret_cast<char*>(p.status) + 1024) +
      ((static_cast<int>(blockIdx.x) * kGroups + group) * 4 + (wave == kConsumers ? 0 : wave + 1)) * 4;
  const int tl_start = static_cast<int>(__builtin_amdgcn_s_memrealtime());
  int tl_first = 0, tl_tiles = 0, tl_items = 0;
  auto tl_now = [] { return static_cast<int>(__builtin_amdgcn_s_memrealtime()); };
  auto tl_write = [&]() {
    if (lane == 0 && blockIdx.x < 256) {
      tl_rec[0] = tl_start; tl_rec[1] = tl_first; tl_rec[2] = tl_now(); tl_rec[3] = tl_tiles | (tl_items << 16);
    }
  };)

  const int R = p.rows;
  // The groups of all workgroups are the workers; worker ids of one workgroup
  // are equal mod 8 when the grid is a multiple of 8.
  const int G = kGroups * static_cast<int>(gridDim.x);
  const int worker = static_cast<int>(blockIdx.x) + group * static_cast<int>(gridDim.x);
  // Work entries of the plan (its merge entries follow them; see the producer).
  // The producer wave asks for its first kListedItems records before anything
  // looks at this count (the index is kept inside the entry array): count and
  // records are in flight together, one memory latency for both.
  const int n_entries = load_uniform(p.status + kStateEntries);
  int4 listed0 = make_int4(-1, 0, 0, 0), listed1 = make_int4(0, 0, 0, 0);
  if (wave == kConsumers) {
    const int j = (lane & 1) ? (G - 1 - worker) : worker;
    const int i = lane * G + j;
    const int entry = ((i >> 3) / a.kv_heads) * 8 + (i & 7);
    const int4* en = reinterpret_cast<const int4*>(p.entries + min(entry, p.total_items / a.kv_heads - 1));
    listed0 = en[0];
    listed1 = en[1];
  }
  const int n_ids = (n_entries + 7) / 8 * 8 * a.kv_heads;  // item ids that may name a work entry
  const int n_rounds = (n_ids + G - 1) / G;
  constexpr bool has_new = NEW != kNewNone;
  // the new token arrives unquantised: the consumer of its tile quantises it
  constexpr bool quant_new = std::is_same<KV, int8_t>::value && NEW >= kNewRaw;
  // more than 16 KV heads: the token's raw rows fill two tiles, keys then values,
  // each spread over the key and the value area; one consumer takes both
  constexpr bool wide_new = quant_new && (NEW == kNewRawWide || NEW == kNewRawWideRope);
  constexpr bool rope_new = quant_new && (NEW == kNewRawRope || NEW == kNewRawWideRope);  // the key is rotated first
  // the new token is also written into its slot's page (paged caches)
  const bool to_pages = PAGED && has_new && a.new_to_pages != 0;

  // Item of round k of this worker: virtual ids k*G + j with j running forwards
  // in even rounds and backwards in odd ones, so that with entries sorted
  // longest first every worker gets a similar total.  Virtual id i maps to
  // (entry, head) with all heads of an entry on ids of equal i % 8: workgroup
  // ids go round-robin over the 8 XCDs, so an entry's scales and page-table
  // row are fetched into one L2 only.  Unused entries give invalid items.
  auto item_index = [&](int k, int* entry, int* h) -> bool {
    const int j = (k & 1) ? (G - 1 - worker) : worker;
    const int i = k * G + j;
    const int m = i >> 3;
    *entry = (m / a.kv_heads) * 8 + (i & 7);
    *h = m % a.kv_heads;
    return k < n_rounds && i < n_ids && *entry < n_entries;
  };
  // The first kListedItems rounds are read here, all at once, into LDS (one
  // memory latency for the lot, and none inside the stream); later rounds, which
  // only very large batches have, are read when they are reached.
  char* const ring = ring_all[group];
  auto& sm_o = sm_o_all[group];
  auto& sm_q = sm_q_all[group];
  auto& sm_qmeta = sm_qmeta_all[group];
  auto& sm_m = sm_m_all[group];
  auto& sm_l = sm_l_all[group];
  int* const sm_filled = sm_filled_all[group];
  int* const sm_freed = sm_freed_all[group];
  int* const sm_qtaken = sm_qtaken_all[group];
  int* const sm_arrived = sm_arrived_all[group];
  int* const sm_folded = sm_folded_all[group];
  int (*const sm_items)[8] = sm_items_all[group];
  int (*const sm_pages)[kStagedPages] = sm_pages_all[PAGED ? group : 0];
  if (wave == kConsumers) {
    int entry, h;
    if (!item_index(lane, &entry, &h)) listed0 = make_int4(-1, 0, 0, 0);
    // slot, start, count, part | n_chunks, head, valid, slot length
    *reinterpret_cast<int4*>(&sm_items[lane][0]) = listed0;
    *reinterpret_cast<int4*>(&sm_items[lane][4]) = make_int4(listed1.x, h, listed0.x >= 0 ? 1 : 0, listed1.y);
  }
  __syncthreads();
  auto unpack_item = [&](int4 e0, int4 e1) -> Item {
    Item it;
    it.slot = __builtin_amdgcn_readfirstlane(e0.x);
    it.start = __builtin_amdgcn_readfirstlane(e0.y);
    it.count = __builtin_amdgcn_readfirstlane(e0.z);
    it.part = __builtin_amdgcn_readfirstlane(e0.w);
    it.n_chunks = __builtin_amdgcn_readfirstlane(e1.x);
    it.h = __builtin_amdgcn_readfirstlane(e1.y);
    it.valid = __builtin_amdgcn_readfirstlane(e1.z) != 0;
    it.len = __builtin_amdgcn_readfirstlane(e1.w);
    return it;
  };
  auto fetch = [&](int k) -> Item {  // rounds past the listed ones
    Item it;
    int entry, h;
    it.valid = item_index(k, &entry, &h);
    it.slot = it.start = it.count = it.part = it.n_chunks = it.h = it.len = 0;
    if (it.valid) {
      const int32_t* en = reinterpret_cast<const int32_t*>(p.entries + entry);
      it.h = h;
      it.slot = load_uniform(en + 0); it.start = load_uniform(en + 1); it.count = load_uniform(en + 2);
      it.part = load_uniform(en + 3); it.n_chunks = load_uniform(en + 4); it.len = load_uniform(en + 5);
      it.valid = it.slot >= 0;
    }
    return it;
  };
  // tiles of an item: its cache positions, plus one for the step's new token
  // on the slot's first chunk (when the token also goes into the pages, an
  // empty slot is an inactive one and has no token)
  auto cache_tiles = [&](const Item& it) { return (it.count + kTile - 1) / kTile; };
  auto item_tiles = [&](const Item& it) {
    return cache_tiles(it) + ((has_new && it.start == 0 && !(to_pages && it.len == 0)) ? (wide_new ? 2 : 1) : 0);
  };
  // A wave gives up: the other waves of the workgroup see the flag at their
  // next wait and leave too, and the host finds the sticky word in the
  // workspace's state block (jpt_attn_status).
  auto give_up = [&]() {
    lds_poke(&sm_abort, 1);
    if (lane == 0) __hip_atomic_fetch_or(p.status, JPT_ATTN_STATUS_GAVE_UP, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  // Bounded wait for an LDS counter; false = give up (abort raised).
  auto wait_for = [&](int* counter, int needed) -> bool {
    int spins = 0;
    while (__hip_atomic_load(counter, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < needed) {
      if (++spins > kSpinLimit ||
          __hip_atomic_load(&sm_abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) {
        give_up();
        return false;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    return true;
  };

  // Partials travel between workgroups on different XCDs, each behind an L2 of
  // its own, without a device-wide fence: they are written through to memory and
  // read from memory past every cache level (system scope).  A row of a partial
  // is written and read 16 bytes a lane with the 16 lanes of a row side by side -
  // float4 number q of lane l at float 64 q + 4 l, so lane l's outputs
  // [8 l, 8 l + 8) are its two float4 - because a wave's store of 256 contiguous
  // bytes is whole memory lines, where one float a lane 32 bytes apart costs a
  // 32-byte memory write each (measured: 7 MB of writes a launch for 0.7 MB of
  // partials).  The row's statistics (max, sum) follow at float 128.
  auto put_row = [](float* row, int lane_in_row, const float (&o)[8], float M, float l) {
    const f32x4 q0 = {o[0], o[1], o[2], o[3]}, q1 = {o[4], o[5], o[6], o[7]};
    float* at = row + 4 * lane_in_row;
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\t"
                 "global_store_dwordx4 %0, %2, off offset:256 sc0 sc1" : : "v"(at), "v"(q0), "v"(q1) : "memory");
    if (lane_in_row == 0) {
      typedef __attribute__((ext_vector_type(2))) float f32x2;
      const f32x2 st = {M, l};
      asm volatile("global_store_dwordx2 %0, %1, off offset:512 sc0 sc1" : : "v"(row), "v"(st) : "memory");
    }
  };
  // Rows of two partials at once (one memory latency for both); the caller's
  // wave has no other loads in flight.
  struct PartRow {
    f32x4 q0, q1;
    __attribute__((ext_vector_type(2))) float st;
  };
  auto get_rows = [](const float* row_a, const float* row_b, int lane_in_row, PartRow& ra, PartRow& rb) {
    const float* at_a = row_a + 4 * lane_in_row;
    const float* at_b = row_b + 4 * lane_in_row;
    asm volatile("global_load_dwordx4 %0, %6, off sc0 sc1\n\t"
                 "global_load_dwordx4 %1, %6, off offset:256 sc0 sc1\n\t"
                 "global_load_dwordx2 %2, %7, off offset:512 sc0 sc1\n\t"
                 "global_load_dwordx4 %3, %8, off sc0 sc1\n\t"
                 "global_load_dwordx4 %4, %8, off offset:256 sc0 sc1\n\t"
                 "global_load_dwordx2 %5, %9, off offset:512 sc0 sc1\n\t"
                 "s_waitcnt vmcnt(0)"
                 : "=&v"(ra.q0), "=&v"(ra.q1), "=&v"(ra.st), "=&v"(rb.q0), "=&v"(rb.q1), "=&v"(rb.st)
                 : "v"(at_a), "v"(row_a), "v"(at_b), "v"(row_b)
                 : "memory");
  };
  // writes rows of outputs: 16 lanes a row, eight outputs a lane, the statistics by the row's first lane
  auto write_row = [&](int64_t q_row, int d0, const float (&o)[8], float M, float l) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    const uint4 packed = make_uint4(pack_bf16(o[0] * inv, o[1] * inv), pack_bf16(o[2] * inv, o[3] * inv),
                                    pack_bf16(o[4] * inv, o[5] * inv), pack_bf16(o[6] * inv, o[7] * inv));
    *reinterpret_cast<uint4*>(static_cast<uint16_t*>(a.out) + q_row * kD + d0) = packed;
    if (d0 == 0) {
      if (a.out_max) a.out_max[q_row] = M * kLn2;
      if (a.out_denom) a.out_denom[q_row] = l;
    }
  };
  // A merge item: every chunk of the slot has parked its partial and been
  // counted (merge entries come last in the plan and the chunks first, so the
  // wait is normally over before it starts; it is bounded like every other);
  // folds the partials and writes the slot's output.  One wave's work.
  auto merge_item = [&](const Item& it) -> bool {
    int32_t* counter = p.arrivals + static_cast<int64_t>(it.slot) * a.kv_heads + it.h;
    // The chunks belong to other workgroups, which must get to run for this wait
    // to end: it is a long one (a poll takes about a microsecond with its sleep:
    // some 60 ms in all), long enough for workgroups held back by other work on
    // the device to be scheduled.
    for (int spins = 0;; ++spins) {
      int seen = 0;
      if (lane == 0) seen = __hip_atomic_fetch_add(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (__builtin_amdgcn_readfirstlane(seen) >= it.n_chunks) break;
      if (spins > kMergeSpinLimit || __hip_atomic_load(&sm_abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) {
        give_up();
        return false;
      }
      __builtin_amdgcn_s_sleep(32);
    }
    const int64_t rec = static_cast<int64_t>(R) * kPartFloats;
    const int64_t step = static_cast<int64_t>(a.kv_heads) * rec;
    const int64_t q_row0 = (static_cast<int64_t>(it.slot) * a.q_heads + it.h * p.rep) * a.q_rows;
    const int d0 = 8 * (lane & 15);
    for (int row = lane >> 4; row < R; row += 4) {
      const float* src = p.partials + (static_cast<int64_t>(it.part) * a.kv_heads + it.h) * rec + row * kPartFloats;
      float M = -INFINITY, L = 0.f;
      float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      for (int c0 = 0; c0 < it.n_chunks; c0 += 2) {  // two chunks a trip to memory
        const bool two = c0 + 1 < it.n_chunks;
        PartRow x[2];
        get_rows(src + c0 * step, src + (two ? c0 + 1 : c0) * step, lane & 15, x[0], x[1]);
        const float m0 = x[0].st[0], m1 = two ? x[1].st[0] : -INFINITY;
        const float Mb = fmaxf(M, fmaxf(m0, m1));
        const float keep_old = M == -INFINITY ? 0.f : fast_exp2(M - Mb);
        L *= keep_old;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] *= keep_old;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          const float mc = c == 0 ? m0 : m1;
          const float f = mc == -INFINITY ? 0.f : fast_exp2(mc - Mb);
          L += x[c].st[1] * f;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            o[i] += x[c].q0[i] * f;
            o[4 + i] += x[c].q1[i] * f;
          }
        }
        M = Mb;
      }
      write_row(q_row0 + row, d0, o, M, L);
    }
    // every chunk was counted before its partial was read: nothing touches the counter any more
    if (lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return true;
  };

  if (wave == kConsumers) {
    // ------------------------------- producer -------------------------------
    constexpr int kPieces = C::kRowBytes / 16;       // 16-byte pieces per row
    constexpr int kRowsPerLoad = 64 / kPieces;       // rows one load instruction covers
    constexpr int kLoadsPerMatrix = C::kTileBytes / 1024;
    // Lane l of load j fills LDS piece slot 64j + l: row t = 64j / kPieces +
    // l / kPieces, piece slot l % kPieces, with the global piece chosen by the
    // bank swizzle.  Rows past the chunk end repeat its last row (keeps every
    // access inside the cache and its contents finite).
    int row_of[kLoadsPerMatrix];
    uint32_t piece_off[kLoadsPerMatrix];
#pragma unroll
    for (int j = 0; j < kLoadsPerMatrix; ++j) {
      row_of[j] = j * kRowsPerLoad + lane / kPieces;
      piece_off[j] = static_cast<uint32_t>(((lane % kPieces) ^ (row_of[j] & (kPieces - 1))) * 16);
    }
    // scales, one load for both rows: float32 - lanes 0..31 k, 32..63 v;
    // bf16 - lanes 0..15 k, 16..31 v (two positions per lane)
    constexpr int kHalf = SCALE == kScaleF32 ? 32 : 16;
    constexpr int kEs = SCALE == kScaleF32 ? 4 : 2;
    const char *scale_lane = nullptr, *new_scale_lane = nullptr;
    if (SCALE) {
      const bool is_v = lane >= kHalf;
      scale_lane = static_cast<const char*>(is_v ? a.v_scale : a.k_scale) + (lane - (is_v ? kHalf : 0)) * 4;
      // the new token's two float32 scales, each repeated over its 32 lanes
      if (SCALE == kScaleF32 && has_new)
        new_scale_lane = static_cast<const char*>(is_v ? a.new_v_scale : a.new_k_scale);
    }
    const int q_loads = (R + 3) / 4;  // load instructions for an item's query rows

    int issued = 0, signalled = 0;        // tiles
    int loads_issued = 0;                 // load instructions, all tiles and query rows
    int sig_base = 0;                     // loads issued up to the last signalled tile
    uint64_t carries_q = 0;               // bit t % 64: query rows were loaded just before tile t
    uint64_t carries_p = 0;               // bit t % 64: a row of page ids was loaded just before tile t
    int fill_slot = 0, fill_round = 0;    // issued % kSlots, issued / kSlots
    int sig_slot = 0, sig_round = 1;      // signalled % kSlots, signalled / kSlots + 1
    // Hands every tile that has landed to the consumers.  Loads complete in
    // order, so with `out` loads still counted as outstanding (the wave's own
    // vector-memory counter, read without waiting) the first
    // loads_issued - out loads are complete.
    // int8 codes meet the query as float16 (see Tile<int8_t>): the rows of an
    // item, which arrive as bf16, are turned into that operand here, once, in
    // place, before the item's first tile is handed over - by the wave with
    // time to spare, not by each consumer.  A row is scaled by the power of two
    // that puts its largest magnitude in [2^13, 2^14) (exact; the power goes
    // into the scores' factor), and the bias term 1152 * sum(q) of the row is
    // summed up.  16 lanes a row, eight elements a lane.
    int q_converted = 0;  // items whose rows have been converted
    auto convert_q = [&](int buf) {
      for (int j = 0; j < q_loads; ++j) {
        const int piece = 64 * j + lane;
        const bool live = piece < R * 16;
        uint16_t* at = &sm_q[buf][0][0] + (live ? piece : 0) * 8;
        const i32x4 raw = lds_peek4(reinterpret_cast<const int*>(at));
        float f[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          f[2 * i] = __uint_as_float(static_cast<uint32_t>(raw[i]) << 16);
          f[2 * i + 1] = __uint_as_float(static_cast<uint32_t>(raw[i]) & 0xffff0000u);
        }
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(f[i]));
        amax = row_max(amax);
        int e = 0;
        if (amax > 0.f && amax < INFINITY) frexpf(amax, &e);
        e = max(e, -100);
        const float up = ldexpf(1.f, 14 - e);
        float qs = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          f[i] *= up;
          qs += f[i];
        }
        qs = row_sum(qs);
        if (live) {
          const i32x4 ops = {static_cast<int>(pack_f16(f[0], f[1])), static_cast<int>(pack_f16(f[2], f[3])),
                             static_cast<int>(pack_f16(f[4], f[5])), static_cast<int>(pack_f16(f[6], f[7]))};
          lds_poke4(at, ops);
          if ((piece & 15) == 0) {
            const i32x2 meta = {__builtin_bit_cast(int, ldexpf(1.f, e - 14)),
                                __builtin_bit_cast(int, -Tile<KV>::kBias * qs)};
            lds_poke2(&sm_qmeta[buf][piece >> 4][0], meta);
          }
        }
      }
    };
    auto signal_landed = [&]() {
      const uint32_t ib = __builtin_amdgcn_s_getreg(0xF807);  // HW_REG_IB_STS, all 32 bits
      const int out = static_cast<int>((ib & 0xF) | (((ib >> 22) & 0x3) << 4));
      const int done = loads_issued - out;
      while (signalled < issued) {
        const int need = sig_base + C::kLoadsPerTile + (((carries_q >> (signalled & 63)) & 1) ? q_loads : 0) +
                         (PAGED ? static_cast<int>((carries_p >> (signalled & 63)) & 1) : 0);
        if (done < need) break;
        if (Tile<KV>::kBias != 0.f && ((carries_q >> (signalled & 63)) & 1)) {
          // the tile's item starts here and its query rows landed before it
          convert_q(q_converted % C::kQBufs);
          ++q_converted;
        }
        // LDS takes a wave's writes in order: the operand is there before this word
        lds_poke(&sm_filled[sig_slot], sig_round);  // every lane stores the same word
        sig_base = need;
        carries_q &= ~(1ull << (signalled & 63));
        if (PAGED) carries_p &= ~(1ull << (signalled & 63));
        ++signalled;
        if (++sig_slot == C::kSlots) { sig_slot = 0; ++sig_round; }
      }
    };
    // Bounded wait with hand-overs going on; false = abort.  Also waits until
    // `room` more loads fit under the load counter's limit of 63.
    auto wait_counter = [&](int* counter, int needed, int room) -> bool {
      for (int spins = 0;; ++spins) {
        signal_landed();
        if (loads_issued - sig_base + room <= 63 && lds_peek_uniform(counter) >= needed) return true;
        if (spins > kSpinLimit || lds_peek_uniform(&sm_abort)) {
          give_up();
          __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
          return false;
        }
        __builtin_amdgcn_s_sleep(1);
      }
    };
    // Bounded wait until the first `target` loads have landed and `room` more
    // fit under the counter's limit; false = abort.
    auto wait_landed = [&](int target, int room) -> bool {
      for (int spins = 0;; ++spins) {
        signal_landed();
        const uint32_t ib = __builtin_amdgcn_s_getreg(0xF807);
        const int out = static_cast<int>((ib & 0xF) | (((ib >> 22) & 0x3) << 4));
        if (loads_issued - out >= target && loads_issued - sig_base + room <= 63) return true;
        if (spins > kSpinLimit || lds_peek_uniform(&sm_abort)) {
          give_up();
          __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
          return false;
        }
        __builtin_amdgcn_s_sleep(1);
      }
    };
    // Paged caches: the first kStagedPages page ids of an item's positions, one
    // 4-byte load a lane, into page buffer `buf`.  `with_next_tile`: the load is
    // counted with the next tile to be issued, like query rows (one such load a
    // tile at most); otherwise the caller waits for it and retires it itself.
    auto stage_pages = [&](const Item& it, int buf, bool with_next_tile) {
      const int idx = min(it.start / a.page_size + lane, a.max_pages - 1);  // stays inside the slot's row
      const int32_t* src = a.page_table + (static_cast<int64_t>(it.slot) * a.max_pages + idx);
      __builtin_amdgcn_global_load_lds((global_ptr)src, (lds_ptr)&sm_pages[buf][0], 4, 0, 0);
      loads_issued += 1;
      if (with_next_tile) carries_p |= 1ull << (issued & 63);
    };
    int staged_round = -1;  // round whose page ids were staged while the round before it was issued
    int staged_ready = 0;   // loads_issued right after that staging load
    // Query rows of the `seq`-th item that has tiles into their buffer: piece
    // 64j + lane of the item's R contiguous 256-byte rows.
    auto issue_q = [&](const Item& it, int seq) -> bool {
      const int buf = seq % C::kQBufs;
      if (!wait_counter(&sm_qtaken[buf], kConsumers * (seq / C::kQBufs), q_loads)) return false;
      const char* qrow = static_cast<const char*>(a.q) +
          ((static_cast<int64_t>(it.slot) * a.q_heads + it.h * p.rep) * a.q_rows) * (kD * 2);
      char* dst = reinterpret_cast<char*>(&sm_q[buf][0][0]);
      for (int j = 0; j < q_loads; ++j) {
        const int piece = 64 * j + lane;
        if (piece < R * 16)
          __builtin_amdgcn_global_load_lds((global_ptr)(qrow + piece * 16), (lds_ptr)(dst + j * 1024), 16, 0, 0);
      }
      loads_issued += q_loads;
      carries_q |= 1ull << (issued & 63);
      return true;
    };

    // Issues the loads of one tile into the next ring slot once the slot's
    // previous tile has been taken, handing over landed tiles meanwhile.  `raw`:
    // the key/value areas receive the first bytes at tk/tv as they lie (the new
    // token's unquantised rows) instead of `valid` swizzled rows.
    auto issue_tile = [&](const char* tk, const char* tv, const char* sc, const float* mk, int valid,
                          bool raw, int raw_k_pieces = 0, int raw_v_pieces = 0) -> bool {
      if (!wait_counter(&sm_freed[fill_slot], fill_round, C::kLoadsPerTile)) return false;
      char* slot = ring + fill_slot * C::kSlotBytes;
      if (raw) {
#pragma unroll
        for (int j = 0; j < kLoadsPerMatrix; ++j) {
          // 16-byte pieces of the rows, clamped to those there are
          const uint32_t off_k = static_cast<uint32_t>(min(64 * j + lane, raw_k_pieces - 1)) * 16;
          const uint32_t off_v = static_cast<uint32_t>(min(64 * j + lane, raw_v_pieces - 1)) * 16;
          __builtin_amdgcn_global_load_lds((global_ptr)(tk + off_k), (lds_ptr)(slot + j * 1024), 16, 0, 0);
          __builtin_amdgcn_global_load_lds((global_ptr)(tv + off_v), (lds_ptr)(slot + C::kTileBytes + j * 1024), 16, 0, 0);
        }
      } else {
#pragma unroll
        for (int j = 0; j < kLoadsPerMatrix; ++j) {
          const uint32_t off = static_cast<uint32_t>(min(row_of[j], valid - 1)) * C::kRowBytes + piece_off[j];
          __builtin_amdgcn_global_load_lds((global_ptr)(tk + off), (lds_ptr)(slot + j * 1024), 16, 0, kStreamOnce);
          __builtin_amdgcn_global_load_lds((global_ptr)(tv + off), (lds_ptr)(slot + C::kTileBytes + j * 1024), 16, 0, kStreamOnce);
        }
      }
      char* side = slot + 2 * C::kTileBytes;
      if (SCALE) {
        if (lane < 2 * kHalf) __builtin_amdgcn_global_load_lds((global_ptr)sc, (lds_ptr)side, 4, 0, kStreamOnce);
      }
      if (MASK) {
        if (lane < kTile) __builtin_amdgcn_global_load_lds((global_ptr)(mk + lane), (lds_ptr)(side + 256), 4, 0, 0);
      }
      ++issued;
      JPT_TL(if (tl_first == 0) tl_first = tl_now(); ++tl_tiles;)
      loads_issued += C::kLoadsPerTile;
      if (++fill_slot == C::kSlots) { fill_slot = 0; ++fill_round; }
      return true;
    };

    int q_seq = 0;  // items with tiles so far: only those have their query rows staged
    for (int k = 0; k < n_rounds; ++k) {
      Item cur;
      if (k < kListedItems) {
        const i32x4 e0 = lds_peek4(&sm_items[k][0]), e1 = lds_peek4(&sm_items[k][4]);
        cur = unpack_item(make_int4(e0[0], e0[1], e0[2], e0[3]), make_int4(e1[0], e1[1], e1[2], e1[3]));
      } else {
        cur = fetch(k);
      }
      if (!cur.valid) continue;
      const int hs = a.scale_heads == 1 ? 0 : cur.h;
      const int n_cache = cache_tiles(cur), nt = item_tiles(cur);
      // rows of the item's first position in the key/value and scale tensors
      const char *kt = nullptr, *vt = nullptr;
      int64_t srow = 0;
      const int first_page = PAGED ? cur.start / a.page_size : 0;
      int page = 0, page_no = -1;  // page id of page number page_no of the slot
      if (PAGED) {
        if (n_cache > 0) {
          // page ids of this item: staged during the previous item, or now
          if (staged_round != k) {
            // not staged ahead: load them now and wait.  Once this load has
            // landed so has every load before it, so every issued tile is
            // handed over and the load can be retired on the spot.
            if (!wait_landed(0, 1)) return;
            stage_pages(cur, k & 1, false);
            if (!wait_landed(loads_issued, 0)) return;
            signal_landed();
            sig_base = loads_issued;
          } else if (!wait_landed(staged_ready, 0)) {
            return;
          }
        }
      } else {
        const int64_t row0 = (static_cast<int64_t>(cur.slot) * a.kv_heads + cur.h) * a.seq + cur.start;
        kt = static_cast<const char*>(a.k) + row0 * C::kRowBytes;
        vt = static_cast<const char*>(a.v) + row0 * C::kRowBytes;
        srow = (static_cast<int64_t>(cur.slot) * a.scale_heads + hs) * a.seq + cur.start;
      }
      // an item's query rows travel ahead of its first tile: loads complete
      // in order, so they are in LDS when any of its tiles is handed over
      if (nt > 0 && !issue_q(cur, q_seq++)) return;
      if (PAGED && k + 1 < n_rounds) {
        // page ids of the next item, so that they have landed when it starts
        Item nxt;
        if (k + 1 < kListedItems) {
          const i32x4 e0 = lds_peek4(&sm_items[k + 1][0]), e1 = lds_peek4(&sm_items[k + 1][4]);
          nxt = unpack_item(make_int4(e0[0], e0[1], e0[2], e0[3]), make_int4(e1[0], e1[1], e1[2], e1[3]));
        } else {
          nxt = fetch(k + 1);
        }
        if (nt > 0 && nxt.valid && nxt.count > 0) {  // nt > 0: a tile of this item follows at once
          if (!wait_landed(0, 1)) return;
          stage_pages(nxt, (k + 1) & 1, true);
          staged_round = k + 1;
          staged_ready = loads_issued;
        }
      }
      // The step's new token is the item's first tile: the consumer that gets it
      // has the rest of the item to make up for the extra work it can carry.
      if (nt > n_cache) {
        const int64_t row = static_cast<int64_t>(cur.slot) * a.kv_heads + cur.h;
        const char* tk = static_cast<const char*>(a.new_k) + row * C::kRowBytes;
        const char* tv = static_cast<const char*>(a.new_v) + row * C::kRowBytes;
        if (quant_new) {  // the bf16 rows of all the slot's heads, copied as they lie
          const int64_t raw = static_cast<int64_t>(cur.slot) * a.kv_heads * (kD * 2);
          tk = static_cast<const char*>(a.new_k_raw) + raw;
          tv = static_cast<const char*>(a.new_v_raw) + raw;
        }
        // float32 scales of the new token come through the ring like any
        // tile's; bf16 ones are read by the consumer, and the tile loads the
        // head of the scale tensors only to keep its load count
        const char* sc = scale_lane;
        if (SCALE == kScaleF32) sc = new_scale_lane + (static_cast<int64_t>(cur.slot) * a.scale_heads + hs) * kEs;
        const float* mk = MASK ? static_cast<const float*>(a.mask) + cur.slot * a.mask_stride_b : nullptr;
        const int pieces = a.kv_heads * (kD / 8);  // of one raw tensor's rows
        if (wide_new) {
          constexpr int kAreaPieces = C::kTileBytes / 16;
          if (!issue_tile(tk, tk + C::kTileBytes, sc, mk, 1, true, kAreaPieces, pieces - kAreaPieces)) return;
          if (!issue_tile(tv, tv + C::kTileBytes, sc, mk, 1, true, kAreaPieces, pieces - kAreaPieces)) return;
        } else if (!issue_tile(tk, tv, sc, mk, 1, quant_new, pieces, pieces)) {
          return;
        }
      }
      for (int ct = 0; ct < n_cache; ++ct) {
        const int t0 = cur.start + ct * kTile;
        const int valid = min(kTile, cur.start + cur.count - t0);
        int64_t ts = srow;
        if (PAGED) {  // a tile never straddles a page
          const int pn = t0 / a.page_size;
          if (pn != page_no) {
            page_no = pn;
            page = pn - first_page < kStagedPages
                       ? lds_peek_uniform(&sm_pages[k & 1][pn - first_page])
                       : load_uniform(a.page_table + (static_cast<int64_t>(cur.slot) * a.max_pages + pn));
            page = min(max(page, 0), a.total_pages - 1);  // whatever the table holds, stay inside the pool
          }
          const int64_t in_pool = static_cast<int64_t>(page) * a.page_size + t0 % a.page_size;
          const int64_t row0 = static_cast<int64_t>(cur.h) * a.total_pages * a.page_size + in_pool;
          kt = static_cast<const char*>(a.k) + row0 * C::kRowBytes;
          vt = static_cast<const char*>(a.v) + row0 * C::kRowBytes;
          ts = static_cast<int64_t>(hs) * a.total_pages * a.page_size + in_pool;
        }
        const float* mk = MASK ? static_cast<const float*>(a.mask) + cur.slot * a.mask_stride_b + t0 : nullptr;
        if (!issue_tile(kt, vt, scale_lane + ts * kEs, mk, valid, false)) return;
        if (!PAGED) {
          kt += kTile * C::kRowBytes;
          vt += kTile * C::kRowBytes;
          srow += kTile;
        }
      }
    }
    for (int spins = 0; signalled < issued; ++spins) {
      signal_landed();
      if (spins > kSpinLimit || lds_peek_uniform(&sm_abort)) {
        give_up();
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        return;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    JPT_TL(tl_write();)
    // Every tile of this worker has landed; its consumers are working off the
    // ring.  The producer now folds split slots: it takes (merge entry, head)
    // pairs from a counter in memory for as long as there are any - the workers
    // that are done first do the merging, which costs the launch no tail.  The
    // workers of workgroups equal mod 8 share one counter and the pairs equal to
    // them mod 8 (a dozen nanoseconds per atomic add on one address: one counter
    // for everybody would queue).  Every worker asks until it is refused once:
    // a launch asks a counter exactly pairs + workers times, and the counter
    // counts modulo that number (a wrapping increment), so it is back where it
    // started when the launch ends, launches that follow one another on a plan
    // need no reset, and the counter never grows.  Whatever value a launch finds
    // in it - one that an aborted launch left behind, say - every merge place is
    // handed out exactly once: the asks walk the whole cycle from wherever it
    // starts, and a value outside the cycle costs the first asker a refusal and
    // puts the counter back to zero.
    const int n_merges = load_uniform(p.status + kStateMerges);
    const int share = worker & 7;
    const int sharers = (G - share + 7) / 8;
    const int pairs = n_merges * a.kv_heads;
    const int my_pairs = pairs > share ? (pairs - share + 7) / 8 : 0;
    const unsigned per_launch = static_cast<unsigned>(my_pairs + sharers);
    unsigned* const hand_out = reinterpret_cast<unsigned*>(p.status + kStateHandOut + share * kStateHandOutStride);
    for (;;) {
      unsigned number = 0;
      if (lane == 0) number = __builtin_amdgcn_atomic_inc32(hand_out, per_launch - 1, __ATOMIC_RELAXED, "agent");
      const unsigned place = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(number)));
      if (place >= static_cast<unsigned>(my_pairs)) break;
      const int pair = share + 8 * static_cast<int>(place);
      const int32_t* en = reinterpret_cast<const int32_t*>(p.entries + n_entries + pair / a.kv_heads);
      Item it;
      it.slot = load_uniform(en + 0); it.start = load_uniform(en + 1); it.count = 0;
      it.part = load_uniform(en + 3); it.n_chunks = load_uniform(en + 4); it.len = load_uniform(en + 5);
      it.h = pair % a.kv_heads;
      it.valid = true;
      if (it.slot < 0 || !merge_item(it)) return;
    }
    return;
  }

  // --------------------------------- consumers ---------------------------------
  const int r = lane & 15, g = lane >> 4;
  int pos[8];  // the lane's eight probability positions inside a tile
#pragma unroll
  for (int i = 0; i < 8; ++i) pos[i] = 4 * g + (i & 3) + 16 * (i >> 2);

  using T = Tile<KV>;
  using Op = typename T::Op;
  const float c2 = a.sm_scale * kLog2e;
  Op qop[4];                // Q^T operand: lane (r, g) holds q[row r][32g + 8kk + i], zero for r >= R
  float c2_row = c2;        // c2 times the power of two taken out of the row's q (int8 codes only)
  f32x4 s_init = {0.f, 0.f, 0.f, 0.f};  // score accumulators start here: minus the bias term of the row
  f32x4 acc[8];             // O^T tile j: acc[j][i] = o[row r][32g + 8i + j]
  f32x4 accw = {0.f, 0.f, 0.f, 0.f};    // sum of the weights fed to the second MFMA (int8 codes only)
  float m_run = -INFINITY;  // log2 units, same in the four lanes of a row
  float l_run = 0.f;        // this lane's share of the row sum

  // Takes tile number `t` of the group's stream out of the ring and
  // accumulates it; `valid` positions of the tile count.
  int cur_slot = 0, cur_h = 0;  // of the item being consumed
  // Quantising the new token of slot cur_slot, whose kv_heads bf16 rows lie one
  // after another in `area` (the tile's key or value area): arithmetic and
  // rounding of jpt_kv_append_quant_i8, each step rounded to the scale dtype.
  // The absmax runs over every head (one scale per token) or over head cur_h;
  // only head cur_h is coded, two elements a lane.  Its codes replace row 0 of
  // the area, in tile layout, and go to the stash; the item of head 0 (every
  // item, with per-head scales) stores the scale.
  // `rope`: NULL, or the slot's (cos, sin) factors: the rows are rotated pair by
  // pair first (keys only), rounded to bf16 as the separate rotary op would.
  // Two steps, so that the key's and the value's reductions overlap: new_absmax
  // leaves the lane's two elements of head cur_h in x0, x1 and returns the
  // lane's share of the absmax; new_encode takes the wave-wide absmax.
  constexpr bool kBf16Math = SCALE == kScaleBF16;
  auto new_absmax = [&](const char* area, const float* rope, float& x0, float& x1) -> float {
    auto rotate = [](float& x, float& y, float c, float s) {
#pragma clang fp contract(off)  // the products are rounded before they are combined
      const float xc = x * c, ys = y * s, xs = x * s, yc = y * c;
      const float re = xc - ys;
      const float im = xs + yc;
      x = round_to_bf16(re);
      y = round_to_bf16(im);
    };
    const uint32_t pair = *reinterpret_cast<const uint32_t*>(area + cur_h * (kD * 2) + lane * 4);
    x0 = __uint_as_float(pair << 16);
    x1 = __uint_as_float(pair & 0xffff0000u);
    if (rope) {  // the lane's elements 2 * lane, 2 * lane + 1 of the head are pair number `lane`
      const float2 cs = *reinterpret_cast<const float2*>(rope + 2 * lane);
      rotate(x0, x1, cs.x, cs.y);
    }
    float m = fmaxf(fabsf(x0), fabsf(x1));
    if (a.scale_heads == 1) {
      for (int at = lane * 32; at < a.kv_heads * (kD * 2); at += 64 * 32) {
        const uint4 r0 = *reinterpret_cast<const uint4*>(area + at);
        const uint4 r1 = *reinterpret_cast<const uint4*>(area + at + 16);
        const uint32_t raw[8] = {r0.x, r0.y, r0.z, r0.w, r1.x, r1.y, r1.z, r1.w};
        float f[16];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          f[2 * i] = __uint_as_float(raw[i] << 16);
          f[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
        }
        if (rope) {  // byte `at` of the rows is element (at % 256) / 2 of its head: eight pairs from there
          const float4* cs4 = reinterpret_cast<const float4*>(rope + (at % (kD * 2)) / 2);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float4 cs = cs4[i];
            rotate(f[4 * i], f[4 * i + 1], cs.x, cs.y);
            rotate(f[4 * i + 2], f[4 * i + 3], cs.z, cs.w);
          }
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) m = fmaxf(m, fabsf(f[i]));
      }
    }
    return m;
  };
  auto new_encode = [&](char* area, int8_t* stash, void* scale_out, float x0, float x1, float m) -> float {
    auto rnd = [](float x) { return kBf16Math ? round_to_bf16(x) : x; };
    if (a.new_rounding == JPT_ROUND_RNE) m = fmaxf(m, rnd(1e-5f));
    const float sc = rnd(m / 127.0f);
    int c0, c1;
    if (a.new_rounding == JPT_ROUND_TRUNC) {
      const float q0 = rnd(x0 / sc), q1 = rnd(x1 / sc);
      c0 = (q0 != q0) ? 0 : static_cast<int>(q0);  // 0/0 -> 0; the cast truncates
      c1 = (q1 != q1) ? 0 : static_cast<int>(q1);
    } else {
      const float inv = rnd(1.0f / sc);
      c0 = static_cast<int>(fminf(fmaxf(rintf(rnd(x0 * inv)), -128.f), 127.f));
      c1 = static_cast<int>(fminf(fmaxf(rintf(rnd(x1 * inv)), -128.f), 127.f));
    }
    const uint16_t codes = static_cast<uint16_t>((c0 & 0xff) | ((c1 & 0xff) << 8));
    // row 0 of the tile: piece p sits at piece slot p ^ 0.  Every lane has read
    // its raw elements before any lane's codes land on them.
    *reinterpret_cast<uint16_t*>(area + lane * 2) = codes;
    *reinterpret_cast<uint16_t*>(stash + (static_cast<int64_t>(cur_slot) * a.kv_heads + cur_h) * kD + lane * 2) = codes;
    if (lane == 0 && (a.scale_heads != 1 || cur_h == 0)) {
      const int64_t si = static_cast<int64_t>(cur_slot) * a.scale_heads + (a.scale_heads == 1 ? 0 : cur_h);
      store_from_f32(scale_out, si, kBf16Math ? JPT_BF16 : JPT_F32, sc);
    }
    return sc;
  };
  // The new token on its way into the slot's page (to_pages): the lane's bytes of
  // its key and value rows and its scales, kept from its tile until the item's
  // other tiles are done, when the page id asked for at the item's start is there.
  constexpr int kLaneBytes = C::kRowBytes / 64;  // 2 (codes) or 4 (bf16)
  uint32_t keep_k = 0, keep_v = 0;
  float keep_ks = 0.f, keep_vs = 0.f;
  bool keep = false;
  // Chunks of split slots.  A chunk's partial must be in memory, where the
  // workgroups of every XCD see it, before the chunk is counted as arrived; the
  // wave that parked it does not wait for that: it sends the count after its
  // next tile (or when it is done), when its stores have long been
  // acknowledged.
  int32_t* owed_arrival = nullptr;  // counter of a chunk this wave parked and has not counted yet
  auto count_parked_chunk = [&]() {
    if (owed_arrival == nullptr) return;
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // the partial's write-through stores are acknowledged
    if (lane == 0) __hip_atomic_fetch_add(owed_arrival, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    owed_arrival = nullptr;
  };
  auto consume_tile = [&](int t, int valid, bool is_new) -> bool {
    // One body for every tile: what only the new token's tile or a chunk's last,
    // partly filled tile need sits behind wave-uniform branches, so that the
    // accumulators live in the same registers whichever way a tile goes.
    const bool partial = valid != kTile;
    const int s = t % C::kSlots;
    if (!wait_for(&sm_filled[s], t / C::kSlots + 1)) return false;
    char* slot = ring + s * C::kSlotBytes;
    const char* side = slot + 2 * C::kTileBytes;
    JPT_TL(if (tl_first == 0) tl_first = tl_now(); ++tl_tiles;)
    float new_ks = 0.f, new_vs = 0.f;
    const bool quant_here = is_new && quant_new;
    if (quant_here) {
      const float* rope = rope_new ? a.new_k_rope + static_cast<int64_t>(cur_slot) * kD : nullptr;
      float k0, k1, v0, v1;
      // the raw value rows: this tile's value area, or all of the next tile
      const char* v_rows = slot + C::kTileBytes;
      const int s2 = (t + 1) % C::kSlots;
      if (wide_new) {
        if (!wait_for(&sm_filled[s2], (t + 1) / C::kSlots + 1)) return false;
        v_rows = ring + s2 * C::kSlotBytes;
      }
      const float mk = new_absmax(slot, rope, k0, k1), mv = new_absmax(v_rows, nullptr, v0, v1);
      if (wide_new && lane == 0)  // the next tile has been read (the release waits for the reads)
        __hip_atomic_fetch_add(&sm_freed[s2], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      const float rk = row_max(mk), rv = row_max(mv);  // both reductions in flight together
      new_ks = new_encode(slot, static_cast<int8_t*>(a.new_k), a.new_k_scale, k0, k1,
                          rows_max(rk));
      new_vs = new_encode(slot + C::kTileBytes, static_cast<int8_t*>(a.new_v),
                          a.new_v_scale, v0, v1, rows_max(rv));
    }
    T tile;
    tile.read(slot, slot + C::kTileBytes, r, g, pos);
    // the lane's positions are 4g..4g+3 and 16+4g..16+4g+3
    float ks[8], vs[8], mk[8];
    if (SCALE == kScaleF32) {
      const float4* sk = reinterpret_cast<const float4*>(side);
      const float4 k0 = sk[g], k1 = sk[4 + g], v0 = sk[8 + g], v1 = sk[12 + g];
      ks[0] = k0.x; ks[1] = k0.y; ks[2] = k0.z; ks[3] = k0.w; ks[4] = k1.x; ks[5] = k1.y; ks[6] = k1.z; ks[7] = k1.w;
      vs[0] = v0.x; vs[1] = v0.y; vs[2] = v0.z; vs[3] = v0.w; vs[4] = v1.x; vs[5] = v1.y; vs[6] = v1.z; vs[7] = v1.w;
    } else if (SCALE == kScaleBF16 && is_new) {
      const int64_t si = static_cast<int64_t>(cur_slot) * a.scale_heads + (a.scale_heads == 1 ? 0 : cur_h);
      const float nks = load_as_f32(a.new_k_scale, si, JPT_BF16);
      const float nvs = load_as_f32(a.new_v_scale, si, JPT_BF16);
#pragma unroll
      for (int i = 0; i < 8; ++i) { ks[i] = nks; vs[i] = nvs; }
    } else if (SCALE == kScaleBF16) {
      const uint2* sk = reinterpret_cast<const uint2*>(side);
      const uint2 k0 = sk[g], k1 = sk[4 + g], v0 = sk[8 + g], v1 = sk[12 + g];
      ks[0] = __uint_as_float(k0.x << 16); ks[1] = __uint_as_float(k0.x & 0xffff0000u);
      ks[2] = __uint_as_float(k0.y << 16); ks[3] = __uint_as_float(k0.y & 0xffff0000u);
      ks[4] = __uint_as_float(k1.x << 16); ks[5] = __uint_as_float(k1.x & 0xffff0000u);
      ks[6] = __uint_as_float(k1.y << 16); ks[7] = __uint_as_float(k1.y & 0xffff0000u);
      vs[0] = __uint_as_float(v0.x << 16); vs[1] = __uint_as_float(v0.x & 0xffff0000u);
      vs[2] = __uint_as_float(v0.y << 16); vs[3] = __uint_as_float(v0.y & 0xffff0000u);
      vs[4] = __uint_as_float(v1.x << 16); vs[5] = __uint_as_float(v1.x & 0xffff0000u);
      vs[6] = __uint_as_float(v1.y << 16); vs[7] = __uint_as_float(v1.y & 0xffff0000u);
    }
    if (quant_here) {
#pragma unroll
      for (int i = 0; i < 8; ++i) { ks[i] = new_ks; vs[i] = new_vs; }
    }
    if (MASK) {
      const float4* smk = reinterpret_cast<const float4*>(side + 256);
      const float4 m0 = smk[g], m1 = smk[4 + g];
      mk[0] = m0.x; mk[1] = m0.y; mk[2] = m0.z; mk[3] = m0.w; mk[4] = m1.x; mk[5] = m1.y; mk[6] = m1.z; mk[7] = m1.w;
      if (is_new) {
#pragma unroll
        for (int i = 0; i < 8; ++i) mk[i] = 0.f;
      }
    }
    if (is_new && to_pages) {  // row 0 of the tile: piece p sits at piece slot p
      if (kLaneBytes == 2) {
        keep_k = *reinterpret_cast<const uint16_t*>(slot + lane * 2);
        keep_v = *reinterpret_cast<const uint16_t*>(slot + C::kTileBytes + lane * 2);
      } else {
        keep_k = *reinterpret_cast<const uint32_t*>(slot + lane * 4);
        keep_v = *reinterpret_cast<const uint32_t*>(slot + C::kTileBytes + lane * 4);
      }
      if (SCALE) {
        keep_ks = ks[0];
        keep_vs = vs[0];
      }
      keep = true;
    }
    // the registers hold the tile: hand the slot back (the release waits for
    // the LDS reads above)
    if (lane == 0)
      __hip_atomic_fetch_add(&sm_freed[s], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);

    f32x4 sa = s_init, sb = s_init;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      sa = T::mfma(tile.k_op(false, kk), qop[kk], sa);
      sb = T::mfma(tile.k_op(true, kk), qop[kk], sb);
    }
    float sc[8];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float x = (i < 4 ? sa[i] : sb[i - 4]) * (SCALE ? ks[i] * c2_row : c2_row);
      if (MASK) x += mk[i] * kLog2e;
      sc[i] = x;
    }
    if (partial) {
#pragma unroll
      for (int i = 0; i < 8; ++i) sc[i] = pos[i] < valid ? sc[i] : -INFINITY;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) tmax = fmaxf(tmax, sc[i]);
    tmax = max_across_rows(tmax);
    const float m_new = fmaxf(m_run, tmax);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_use);
    float w[8], psum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float pr = fast_exp2(sc[i] - m_use);
      psum += pr;
      w[i] = SCALE ? pr * vs[i] : pr;
    }
    if (SCALE && partial) {  // a position that does not count has weight 0 whatever its scale holds
#pragma unroll
      for (int i = 0; i < 8; ++i) w[i] = pos[i] < valid ? w[i] : 0.f;
    }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (__any(alpha != 1.f)) {  // rare once the running maximum has settled
      asm volatile("" ::: "memory");  // keeps the compiler from running this speculatively
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] *= alpha;
      if (T::kBias != 0.f) accw *= alpha;
    }
    const Op pop = as_op<Op>(T::pack(w[0], w[1]), T::pack(w[2], w[3]), T::pack(w[4], w[5]), T::pack(w[6], w[7]));
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = T::mfma(tile.v_op(j), pop, acc[j]);
    if (T::kBias != 0.f) accw = T::mfma(T::ones(), pop, accw);
    count_parked_chunk();
    return true;
  };

  // Delivers the wave's part of item number `seq` of this group; the last
  // consumer to arrive folds the parts and writes the slot's output (one
  // chunk) or parks the chunk's partial (several).
  auto finish_item = [&](const Item& it, int seq) -> bool {
    count_parked_chunk();
    const int buf = seq % C::kFoldBufs;
    // the buffer's previous item must have been folded out of it
    if (!wait_for(&sm_folded[buf], seq / C::kFoldBufs)) return false;
    const float l_row = sum_across_rows(l_run);
    if (r < R) {
      const float bias = T::kBias * accw[0];  // every element of accw is the row's weight sum
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) sm_o[buf][wave][r][o_col(32 * g + 8 * i + j)] = acc[j][i] - bias;
      if (g == 0) {
        sm_m[buf][wave][r] = m_run;
        sm_l[buf][wave][r] = l_row;
      }
    }
    int arrived = 0;
    if (lane == 0)
      arrived = __hip_atomic_fetch_add(&sm_arrived[buf], 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
    arrived = __builtin_amdgcn_readfirstlane(arrived);
    if (arrived != kConsumers - 1) return true;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    // Paired chunks (part < 0): the two chunks of a slot cut in two run on the
    // two groups of this workgroup, as the same item of both (the planner puts
    // them on the same round, and every round before it is full).  Group 1
    // leaves its consumers' parts in its fold buffer and says so; group 0 folds
    // both groups' parts, writes the slot's output and frees both buffers.
    const bool pair = it.n_chunks > 1 && it.part < 0;
    if (pair && group == 1) {
      if (lane == 0) __hip_atomic_store(&sm_pair_ready[buf], seq + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      return true;
    }
    if (pair && !wait_for(&sm_pair_ready[buf], seq + 1)) return false;
    const int64_t q_row0 = (static_cast<int64_t>(it.slot) * a.q_heads + it.h * p.rep) * a.q_rows;
    float* part = p.partials + (static_cast<int64_t>(pair ? 0 : it.part) * a.kv_heads + it.h) * R * kPartFloats;
    // four rows a pass: 16 lanes a row, eight consecutive outputs a lane
    const int d0 = 8 * (lane & 15);
    const int n_groups = pair ? 2 : 1;  // whose parts are folded: this group's, then (paired) group 1's
    for (int row = lane >> 4; row < R; row += 4) {
      float M = -INFINITY;
      for (int gi = 0; gi < n_groups; ++gi) {
        const auto& mm = sm_m_all[gi == 0 ? group : 1];
#pragma unroll
        for (int w2 = 0; w2 < kConsumers; ++w2) M = fmaxf(M, mm[buf][w2][row]);
      }
      float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      float l = 0.f;
      for (int gi = 0; gi < n_groups; ++gi) {
        const auto& mm = sm_m_all[gi == 0 ? group : 1];
        const auto& ll = sm_l_all[gi == 0 ? group : 1];
        const auto& oo = sm_o_all[gi == 0 ? group : 1];
#pragma unroll
        for (int w2 = 0; w2 < kConsumers; ++w2) {
          const float mw = mm[buf][w2][row];
          const float f = mw == -INFINITY ? 0.f : fast_exp2(mw - M);
          l += ll[buf][w2][row] * f;
          const float4* src = reinterpret_cast<const float4*>(&oo[buf][w2][row][o_col(d0)]);
          const float4 x = src[0], y = src[1];
          o[0] += x.x * f; o[1] += x.y * f; o[2] += x.z * f; o[3] += x.w * f;
          o[4] += y.x * f; o[5] += y.y * f; o[6] += y.z * f; o[7] += y.w * f;
        }
      }
      if (it.n_chunks == 1 || pair) {
        write_row(q_row0 + row, d0, o, M, l);
      } else {  // park the chunk's partial where the workgroups of every XCD see it
        put_row(part + row * kPartFloats, lane & 15, o, M, l);
      }
    }
    if (it.n_chunks > 1 && !pair) owed_arrival = p.arrivals + static_cast<int64_t>(it.slot) * a.kv_heads + it.h;
    if (lane == 0) {
      __hip_atomic_store(&sm_arrived[buf], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __hip_atomic_fetch_add(&sm_folded[buf], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      if (pair) {
        __hip_atomic_store(&sm_arrived_all[1][buf], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        __hip_atomic_fetch_add(&sm_folded_all[1][buf], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
    return true;
  };

  int base = 0;   // stream number of the current item's tile 0
  int q_seq = 0;  // items with tiles so far
  int seq = 0;    // valid items so far
  for (int k = 0; k < n_rounds; ++k) {
    Item cur;
    if (k < kListedItems) {
      const int4 e0 = *reinterpret_cast<const int4*>(&sm_items[k][0]);
      const int4 e1 = *reinterpret_cast<const int4*>(&sm_items[k][4]);
      cur = unpack_item(e0, e1);
    } else {
      cur = fetch(k);
    }
    if (!cur.valid) continue;
    const int n_cache = cache_tiles(cur), nt = item_tiles(cur);
    if (nt > 0) {
      // query rows: staged by the producer ahead of the item's first tile
      if (!wait_for(&sm_filled[base % C::kSlots], base / C::kSlots + 1)) return;
      const int qb = q_seq++ % C::kQBufs;
      uint4 u[4];
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        u[kk] = make_uint4(0, 0, 0, 0);
        if (r < R) u[kk] = *reinterpret_cast<const uint4*>(&sm_q[qb][r][32 * g + 8 * kk]);
      }
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) qop[kk] = __builtin_bit_cast(Op, u[kk]);
      if (T::kBias != 0.f) {
        // float16 operand made by the producer, with the row's power of two and
        // the bias term of its scores beside it
        float2 meta = make_float2(1.f, 0.f);
        if (r < R) meta = *reinterpret_cast<const float2*>(&sm_qmeta[qb][r][0]);
        c2_row = c2 * meta.x;
        s_init = f32x4{meta.y, meta.y, meta.y, meta.y};
      }
      // taken (the release waits for the reads above)
      if (lane == 0)
        __hip_atomic_fetch_add(&sm_qtaken[qb], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    cur_slot = cur.slot;
    cur_h = cur.h;
    // where the new token goes: the page of position cur.len (asked for now, used
    // after the item's tiles)
    int dst_page = 0;
    const bool dst_room = cur.len < a.max_pages * a.page_size;
    if (to_pages && cur.start == 0 && cur.len > 0 && dst_room)
      dst_page = a.page_table[static_cast<int64_t>(cur.slot) * a.max_pages + cur.len / a.page_size];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    accw = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run = -INFINITY;
    l_run = 0.f;
    // this consumer's tiles: stream numbers congruent to its index
    for (int ti = (wave + kConsumers - base % kConsumers) % kConsumers; ti < nt; ti += kConsumers) {
      if (wide_new && ti == 1 && nt - n_cache == 2) continue;  // read by the consumer of tile 0
      const bool is_new = ti < nt - n_cache;  // the new token comes first
      const int valid = is_new ? 1 : min(kTile, cur.count - (ti - (nt - n_cache)) * kTile);
      if (!consume_tile(base + ti, valid, is_new)) return;
    }
    if (keep) {  // this consumer had the new token's tile
      keep = false;
      if (dst_room && dst_page >= 0) {  // a negative id: the allocator had no page for this token
        const int page = min(dst_page, a.total_pages - 1);  // whatever the table holds, stay inside the pool
        const int64_t in_pool = static_cast<int64_t>(page) * a.page_size + cur.len % a.page_size;
        const int64_t row = static_cast<int64_t>(cur.h) * a.total_pages * a.page_size + in_pool;
        char* dk = static_cast<char*>(a.k) + row * C::kRowBytes + lane * kLaneBytes;
        char* dv = static_cast<char*>(a.v) + row * C::kRowBytes + lane * kLaneBytes;
        if (kLaneBytes == 2) {
          *reinterpret_cast<uint16_t*>(dk) = static_cast<uint16_t>(keep_k);
          *reinterpret_cast<uint16_t*>(dv) = static_cast<uint16_t>(keep_v);
        } else {
          *reinterpret_cast<uint32_t*>(dk) = keep_k;
          *reinterpret_cast<uint32_t*>(dv) = keep_v;
        }
        if (SCALE && lane == 0 && (a.scale_heads != 1 || cur.h == 0)) {
          const int64_t si = static_cast<int64_t>(a.scale_heads == 1 ? 0 : cur.h) * a.total_pages * a.page_size + in_pool;
          store_from_f32(a.k_scale, si, kBf16Math ? JPT_BF16 : JPT_F32, keep_ks);
          store_from_f32(a.v_scale, si, kBf16Math ? JPT_BF16 : JPT_F32, keep_vs);
        }
      }
    }
    JPT_TL(++tl_items;)
    if (!finish_item(cur, seq++)) return;
    base += nt;
  }
  count_parked_chunk();
  JPT_TL(tl_write();)
}

// `workers` groups are wanted; a workgroup holds kGroups of them.
template <typename KV, bool PAGED, int SCALE, bool MASK, int NEW>
void launch_rows(const FastParams& p, unsigned workers, hipStream_t stream) {
  const unsigned blocks = workers / kGroups > 0 ? workers / kGroups : 1;
  if (p.rows <= 4)
    hipLaunchKernelGGL((attn_decode_kernel<KV, PAGED, SCALE, MASK, 4, NEW>), dim3(blocks), dim3(kThreads), 0, stream, p);
  else if (p.rows <= 8)
    hipLaunchKernelGGL((attn_decode_kernel<KV, PAGED, SCALE, MASK, 8, NEW>), dim3(blocks), dim3(kThreads), 0, stream, p);
  else
    hipLaunchKernelGGL((attn_decode_kernel<KV, PAGED, SCALE, MASK, 16, NEW>), dim3(blocks), dim3(kThreads), 0, stream, p);
}

template <typename KV, bool PAGED, int SCALE, int NEW>
void launch_masked(const FastParams& p, unsigned blocks, hipStream_t stream) {
  if (!PAGED && p.a.mask) launch_rows<KV, PAGED, SCALE, !PAGED, NEW>(p, blocks, stream);
  else launch_rows<KV, PAGED, SCALE, false, NEW>(p, blocks, stream);
}

// One translation unit per (cache type, NEW) instantiates this: the kernels of one unit take
// about a minute to compile, and the units compile side by side.  int8 caches come with scales
// (float32 or bf16), bf16 caches without: nothing else is built (attn_fast_supported).
template <typename KV, int NEW>
void launch_decode(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream) {
  if constexpr (std::is_same<KV, int8_t>::value) {
    const bool f32 = p.a.scale_dtype == JPT_F32;
    if (paged) {
      if (f32) launch_masked<KV, true, kScaleF32, NEW>(p, blocks, stream);
      else launch_masked<KV, true, kScaleBF16, NEW>(p, blocks, stream);
    } else {
      if (f32) launch_masked<KV, false, kScaleF32, NEW>(p, blocks, stream);
      else launch_masked<KV, false, kScaleBF16, NEW>(p, blocks, stream);
    }
  } else {
    if (paged) launch_masked<KV, true, kNoScale, NEW>(p, blocks, stream);
    else launch_masked<KV, false, kNoScale, NEW>(p, blocks, stream);
  }
}

}  // namespace decode
}  // namespace jpt
