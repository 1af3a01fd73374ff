// Streaming GQA decode attention kernel for gfx950, head_dim 128 (template
// body; attn_decode_i8.hip and attn_decode_bf16.hip instantiate it).
//
// A persistent workgroup of four wavefronts walks its share of the planned
// (chunk, KV head) items as one stream of 32-position tiles:
//
//   producer wave   copies each tile's K rows, V rows and per-position scales
//                   from HBM straight into an LDS ring with direct-to-LDS
//                   loads (no registers), several tiles ahead and regardless
//                   of item boundaries.  HBM sees full 1 KiB bursts of
//                   contiguous cache rows; a first touch of a new cache row
//                   (several microseconds with its TLB miss) is hidden behind
//                   the tiles already in the ring.
//   consumer waves  take tiles round-robin out of the ring, convert int8 codes
//                   to bf16 in registers (exact) and run
//                       S^T = K . Q^T   v_mfma_f32_16x16x32_bf16, positions on
//                                       M, the rep*q_rows query rows on N
//                       O^T = V^T . P^T positions on the contraction index
//                   with an online softmax in between.  The score
//                   accumulators of lane (row r, group g) are exactly the
//                   probabilities that lane feeds to the second MFMA, so
//                   probabilities never cross lanes.
//
// Waves never meet at a workgroup barrier: ring slots are handed over through
// LDS counters, and the consumer that delivers the last part of an item folds
// the three parts and writes the slot's output (one chunk) or parks the
// chunk's float32 partial (several; a second kernel folds those).  Every wait
// is bounded: a wave that waits too long raises an abort flag and every wave
// leaves, so a logic error shows up as wrong output, never as a hung GPU.
#pragma once

#include <math.h>

#include "attn_common.h"
#include "attn_plan.h"

namespace jpt {
namespace decode {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef const __attribute__((address_space(1))) void* global_ptr;
typedef __attribute__((address_space(3))) void* lds_ptr;

#ifndef JPT_ATTN_CONSUMERS
#define JPT_ATTN_CONSUMERS 3
#endif
#ifndef JPT_ATTN_WAVES_PER_SIMD
#define JPT_ATTN_WAVES_PER_SIMD 2
#endif
constexpr int kConsumers = JPT_ATTN_CONSUMERS;
constexpr int kWaves = kConsumers + 1;
constexpr int kThreads = kWaves * 64;
constexpr int kSideBytes = 512;     // ks | vs | mask, 128 bytes each at most
constexpr int kOStride = 140;       // padded LDS row of 128 outputs
constexpr int kLdsBudget = 80 * 1024 - 256;  // two workgroups per compute unit
constexpr int kSpinLimit = 1 << 18;  // tens of milliseconds
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
  static constexpr int kFoldBufs = ((RC > 8 && kElem > 1) || kConsumers > 3) ? 1 : 2;
  static constexpr int kFoldBytes = kFoldBufs * kConsumers * RC * (kOStride + 2) * 4;
  static constexpr int kSlotsByLds = (kLdsBudget - kFoldBytes) / kSlotBytes;
  static constexpr int kSlotsByCount = 63 / kLoadsPerTile;  // the load counter counts to 63
  // ring slots: every one may hold a tile in flight
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
__device__ __forceinline__ void lds_poke(int* p, int v) {
  const uint32_t addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_int_ptr)p));
  asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(v) : "memory");
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

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding)
constexpr int vmcnt_imm(int n) { return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14); }

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  bf16x2 t = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
  return __builtin_bit_cast(uint32_t, t);
}
__device__ __forceinline__ float sbyte(uint32_t w, int k) {
  return static_cast<float>(static_cast<signed char>(w >> (8 * k)));
}
__device__ __forceinline__ bf16x8 as_op(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  uint4 u = make_uint4(a, b, c, d);
  return __builtin_bit_cast(bf16x8, u);
}

// One tile in a consumer's registers.  Lane (r, g) holds elements [32g, 32g+32)
// of positions r and 16+r (K) and elements [8r, 8r+8) of its eight probability
// positions (V).  In LDS a row is stored as 16-byte pieces, piece p of
// position t at piece slot p ^ (t & 7) (int8) or p ^ (t & 15) (bf16), which
// spreads both access patterns over the banks.
template <typename KV>
struct Tile;

template <>
struct Tile<int8_t> {
  uint4 ka[2], kb[2];
  uint2 v[8];
  __device__ __forceinline__ void read(const char* ks, const char* vs, int r, int g, const int* pos) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int t = r + 16 * half;
      const uint4* row = reinterpret_cast<const uint4*>(ks + t * 128);
      const uint4 x = row[(2 * g) ^ (t & 7)], y = row[(2 * g + 1) ^ (t & 7)];
      if (half == 0) { ka[0] = x; ka[1] = y; } else { kb[0] = x; kb[1] = y; }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int t = pos[i];
      v[i] = *reinterpret_cast<const uint2*>(vs + t * 128 + 16 * ((r >> 1) ^ (t & 7)) + 8 * (r & 1));
    }
  }
  __device__ __forceinline__ bf16x8 k_op(bool second, int kk) const {
    const uint4& q = second ? kb[kk >> 1] : ka[kk >> 1];
    const uint32_t w0 = (kk & 1) ? q.z : q.x, w1 = (kk & 1) ? q.w : q.y;
    return as_op(pack_bf16(sbyte(w0, 0), sbyte(w0, 1)), pack_bf16(sbyte(w0, 2), sbyte(w0, 3)),
                 pack_bf16(sbyte(w1, 0), sbyte(w1, 1)), pack_bf16(sbyte(w1, 2), sbyte(w1, 3)));
  }
  __device__ __forceinline__ float v_elem(int i, int j) const {
    return sbyte(j < 4 ? v[i].x : v[i].y, j & 3);
  }
  __device__ __forceinline__ bf16x8 v_op(int j) const {
    return as_op(pack_bf16(v_elem(0, j), v_elem(1, j)), pack_bf16(v_elem(2, j), v_elem(3, j)),
                 pack_bf16(v_elem(4, j), v_elem(5, j)), pack_bf16(v_elem(6, j), v_elem(7, j)));
  }
};

template <>
struct Tile<__bf16> {
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
  __device__ __forceinline__ bf16x8 k_op(bool second, int kk) const {
    return __builtin_bit_cast(bf16x8, second ? kb[kk] : ka[kk]);
  }
  __device__ __forceinline__ uint32_t v_word(int i, int j) const {
    const int w = j >> 1;
    return w == 0 ? v[i].x : w == 1 ? v[i].y : w == 2 ? v[i].z : v[i].w;
  }
  __device__ __forceinline__ bf16x8 v_op(int j) const {
    const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
    return as_op(__builtin_amdgcn_perm(v_word(1, j), v_word(0, j), sel),
                 __builtin_amdgcn_perm(v_word(3, j), v_word(2, j), sel),
                 __builtin_amdgcn_perm(v_word(5, j), v_word(4, j), sel),
                 __builtin_amdgcn_perm(v_word(7, j), v_word(6, j), sel));
  }
};

// Per-wave timing records for development builds (-DJPT_ATTN_TRACE): eight
// 64-bit words per wave, times in ticks of the 100 MHz real-time counter.
#ifdef JPT_ATTN_TRACE
#define JPT_TR(stmt) stmt
#else
#define JPT_TR(stmt)
#endif

// One work item: a chunk of one slot for one KV head.
struct Item {
  int slot, start, count, part, n_chunks, h;
  bool valid;
};

template <typename KV, bool PAGED, int SCALE, bool MASK, int RC>
__global__ void __launch_bounds__(kThreads, JPT_ATTN_WAVES_PER_SIMD) attn_decode_kernel(FastParams p) {
  using C = Config<KV, SCALE, MASK, RC>;
  const jpt_attn_args& a = p.a;
  __shared__ __attribute__((aligned(1024))) char ring[C::kSlots * C::kSlotBytes];
  __shared__ __attribute__((aligned(16))) float sm_o[C::kFoldBufs][kConsumers][RC][kOStride];
  __shared__ float sm_m[C::kFoldBufs][kConsumers][RC];
  __shared__ float sm_l[C::kFoldBufs][kConsumers][RC];
  __shared__ int sm_filled[C::kSlots];   // times the producer filled this slot
  __shared__ int sm_freed[C::kSlots];    // times a consumer emptied it
  __shared__ int sm_arrived[C::kFoldBufs];
  __shared__ int sm_folded[C::kFoldBufs];
  __shared__ int sm_abort;

  __shared__ int sm_simd[kWaves];
  const int tid = threadIdx.x, lane = tid & 63;
  const int hw_wave = tid >> 6;
  JPT_TR(const unsigned long long tr_start = __builtin_amdgcn_s_memrealtime();)
  JPT_TR(unsigned long long tr_wait = 0; unsigned long long tr_fold = 0; unsigned long long tr_first = 0; unsigned long long tr_t = 0; int tr_tiles = 0;)
  if (tid < C::kSlots) { sm_filled[tid] = 0; sm_freed[tid] = 0; }
  if (tid < C::kFoldBufs) { sm_arrived[tid] = 0; sm_folded[tid] = 0; }
  if (tid == 0) sm_abort = 0;
  if (lane == 0) sm_simd[hw_wave] = (__builtin_amdgcn_s_getreg(0xF804) >> 4) & 3;  // HW_REG_HW_ID: SIMD_ID
  __syncthreads();
  // Roles.  The producer is nearly idle, so the two workgroups sharing a
  // compute unit should not both park theirs on the same SIMD: pick the wave
  // that runs on a SIMD derived from the workgroup id (workgroups j and j+32
  // of an XCD share a unit), if there is one.  `wave` is the role index:
  // consumers 0..kConsumers-1, producer kConsumers.
  int producer_wave;
  {
    const int j = blockIdx.x >> 3;
    const int want = (((j >> 5) & 1) << 1) | (j & 1);
    producer_wave = want % kWaves;
    for (int w = kWaves - 1; w >= 0; --w)
      if (sm_simd[w] == want) producer_wave = w;
  }
  const int wave = hw_wave == producer_wave ? kConsumers : hw_wave - (hw_wave > producer_wave ? 1 : 0);

  const int R = p.rows;
  const int G = gridDim.x;  // multiple of 8
  const bool has_new = a.new_k != nullptr;

  // Item sequence of this workgroup: virtual ids k*G + j with j running
  // forwards in even rounds and backwards in odd ones, so that with entries
  // sorted longest first every workgroup gets a similar total.  Virtual id i
  // maps to (entry, head) with all heads of an entry on ids of equal i % 8:
  // workgroup ids go round-robin over the 8 XCDs, so an entry's scales and
  // page-table row are fetched into one L2 only.
  auto fetch = [&](int k) -> Item {
    Item it;
    const int j = (k & 1) ? (G - 1 - static_cast<int>(blockIdx.x)) : static_cast<int>(blockIdx.x);
    const int i = k * G + j;
    it.valid = i < p.total_items;
    it.slot = it.start = it.count = it.part = it.n_chunks = it.h = 0;
    if (it.valid) {
      const int m = i >> 3;
      const int32_t* en = reinterpret_cast<const int32_t*>(p.entries + ((m / a.kv_heads) * 8 + (i & 7)));
      it.h = m % a.kv_heads;
      it.slot = load_uniform(en + 0); it.start = load_uniform(en + 1); it.count = load_uniform(en + 2);
      it.part = load_uniform(en + 3); it.n_chunks = load_uniform(en + 4);
      it.valid = it.slot >= 0;
    }
    return it;
  };
  // tiles of an item: its cache positions, plus one for the step's new token
  // on the slot's first chunk
  auto cache_tiles = [&](const Item& it) { return (it.count + kTile - 1) / kTile; };
  auto item_tiles = [&](const Item& it) {
    return cache_tiles(it) + ((has_new && it.start == 0) ? 1 : 0);
  };
  // Bounded wait for an LDS counter; false = give up (abort raised).
  auto wait_for = [&](int* counter, int needed) -> bool {
    int spins = 0;
    while (__hip_atomic_load(counter, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < needed) {
      if (++spins > kSpinLimit ||
          __hip_atomic_load(&sm_abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) {
        __hip_atomic_store(&sm_abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        return false;
      }
      __builtin_amdgcn_s_sleep(1);
    }
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
    const char* scale_lane = nullptr;
    if (SCALE) {
      const bool is_v = lane >= kHalf;
      scale_lane = static_cast<const char*>(is_v ? a.v_scale : a.k_scale) + (lane - (is_v ? kHalf : 0)) * 4;
    }
    constexpr int kEs = SCALE == kScaleF32 ? 4 : 2;

    int issued = 0, signalled = 0;
    int fill_slot = 0, fill_round = 0;    // issued % kSlots, issued / kSlots
    int sig_slot = 0, sig_round = 1;      // signalled % kSlots, signalled / kSlots + 1
    // Hands every tile that has landed to the consumers.  Loads complete in
    // order, so with `out` loads still counted as outstanding (the wave's own
    // vector-memory counter, read without waiting) all tiles but the newest
    // ceil(out / loads-per-tile) are complete.
    auto signal_landed = [&]() {
      const uint32_t ib = __builtin_amdgcn_s_getreg(0xF807);  // HW_REG_IB_STS, all 32 bits
      const int out = static_cast<int>((ib & 0xF) | (((ib >> 22) & 0x3) << 4));
      const int landed = issued - (out + C::kLoadsPerTile - 1) / C::kLoadsPerTile;
      while (signalled < landed) {
        if (lane == 0) lds_poke(&sm_filled[sig_slot], sig_round);
        ++signalled;
        if (++sig_slot == C::kSlots) { sig_slot = 0; ++sig_round; }
      }
    };
    Item cur = fetch(0);
    Item nxt = fetch(1);
    for (int k = 0; cur.valid; ++k) {
      const Item nxt2 = fetch(k + 2);  // entries are read two items ahead of their use
      const int hs = a.scale_heads == 1 ? 0 : cur.h;
      const int n_cache = cache_tiles(cur), nt = item_tiles(cur);
      // rows of the item's first position in the key/value and scale tensors
      const char *kt = nullptr, *vt = nullptr;
      int64_t srow = 0;
      int page = 0;
      if (PAGED) {
        page = load_uniform(a.page_table + (static_cast<int64_t>(cur.slot) * a.max_pages + cur.start / a.page_size));
      } else {
        const int64_t row0 = (static_cast<int64_t>(cur.slot) * a.kv_heads + cur.h) * a.seq + cur.start;
        kt = static_cast<const char*>(a.k) + row0 * C::kRowBytes;
        vt = static_cast<const char*>(a.v) + row0 * C::kRowBytes;
        srow = (static_cast<int64_t>(cur.slot) * a.scale_heads + hs) * a.seq + cur.start;
      }
      for (int ti = 0; ti < nt; ++ti) {
        const bool is_new = ti >= n_cache;
        int valid = 1;  // the new token: every row of the tile is that one token
        if (is_new) {
          const int64_t row = static_cast<int64_t>(cur.slot) * a.kv_heads + cur.h;
          kt = static_cast<const char*>(a.new_k) + row * C::kRowBytes;
          vt = static_cast<const char*>(a.new_v) + row * C::kRowBytes;
          srow = 0;  // its scales are read by the consumers; load the tensors' heads
        } else {
          const int t0 = cur.start + ti * kTile;
          valid = min(kTile, cur.start + cur.count - t0);
          if (PAGED) {  // a tile never straddles a page
            const int64_t in_pool = static_cast<int64_t>(page) * a.page_size + t0 % a.page_size;
            const int64_t row0 = static_cast<int64_t>(cur.h) * a.total_pages * a.page_size + in_pool;
            kt = static_cast<const char*>(a.k) + row0 * C::kRowBytes;
            vt = static_cast<const char*>(a.v) + row0 * C::kRowBytes;
            srow = static_cast<int64_t>(hs) * a.total_pages * a.page_size + in_pool;
            // page of the next tile, read while this one is issued
            const int tn = min(t0 + kTile, cur.start + cur.count - 1);
            page = load_uniform(a.page_table + (static_cast<int64_t>(cur.slot) * a.max_pages + tn / a.page_size));
          }
        }
        // wait for the slot's previous tile to be taken, handing over landed
        // tiles meanwhile
        JPT_TR(tr_t = __builtin_amdgcn_s_memrealtime();)
        for (int spins = 0;; ++spins) {
          signal_landed();
          if (lds_peek(&sm_freed[fill_slot]) >= fill_round) break;
          if (spins > kSpinLimit || lds_peek(&sm_abort)) {
            lds_poke(&sm_abort, 1);
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            return;
          }
          __builtin_amdgcn_s_sleep(1);
        }
        JPT_TR(tr_wait += __builtin_amdgcn_s_memrealtime() - tr_t; if (!tr_first) tr_first = __builtin_amdgcn_s_memrealtime() - tr_start;)
        char* slot = ring + fill_slot * C::kSlotBytes;
#pragma unroll
        for (int j = 0; j < kLoadsPerMatrix; ++j) {
          const uint32_t off = static_cast<uint32_t>(min(row_of[j], valid - 1)) * C::kRowBytes + piece_off[j];
          __builtin_amdgcn_global_load_lds((global_ptr)(kt + off), (lds_ptr)(slot + j * 1024), 16, 0, 0);
          __builtin_amdgcn_global_load_lds((global_ptr)(vt + off), (lds_ptr)(slot + C::kTileBytes + j * 1024), 16, 0, 0);
        }
        char* side = slot + 2 * C::kTileBytes;
        if (SCALE) {
          if (lane < 2 * kHalf)
            __builtin_amdgcn_global_load_lds((global_ptr)(scale_lane + srow * kEs), (lds_ptr)side, 4, 0, 0);
        }
        if (MASK) {
          const float* src = static_cast<const float*>(a.mask) + cur.slot * a.mask_stride_b + (is_new ? 0 : cur.start + ti * kTile);
          if (lane < kTile)
            __builtin_amdgcn_global_load_lds((global_ptr)(src + lane), (lds_ptr)(side + 256), 4, 0, 0);
        }
        ++issued;
        if (++fill_slot == C::kSlots) { fill_slot = 0; ++fill_round; }
        if (!PAGED) {
          kt += kTile * C::kRowBytes;
          vt += kTile * C::kRowBytes;
          srow += kTile;
        }
      }
      cur = nxt;
      nxt = nxt2;
    }
    for (int spins = 0; signalled < issued; ++spins) {
      signal_landed();
      if (spins > kSpinLimit || lds_peek(&sm_abort)) {
        lds_poke(&sm_abort, 1);
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        return;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    JPT_TR(if (p.trace && lane == 0) {
      unsigned long long* o = p.trace + (static_cast<size_t>(blockIdx.x) * kWaves + wave) * 8;
      o[0] = issued; o[1] = tr_wait; o[2] = 0; o[3] = __builtin_amdgcn_s_memrealtime() - tr_start;
      o[4] = tr_start; o[5] = 0; o[6] = tr_first; o[7] = sm_simd[hw_wave];
    })
    return;
  }

  // --------------------------------- consumers ---------------------------------
  const int r = lane & 15, g = lane >> 4;
  int pos[8];  // the lane's eight probability positions inside a tile
#pragma unroll
  for (int i = 0; i < 8; ++i) pos[i] = 4 * g + (i & 3) + 16 * (i >> 2);

  // Q^T operand: lane (r, g) holds q[row r][32g + 8kk + i], zero for r >= R
  auto load_q = [&](bf16x8* qop, const Item& it) {
    const char* qrow = static_cast<const char*>(a.q) +
        ((static_cast<int64_t>(it.slot) * a.q_heads + it.h * p.rep) * a.q_rows + r) * (kD * 2);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      uint4 u = make_uint4(0, 0, 0, 0);
      if (r < R) u = *reinterpret_cast<const uint4*>(qrow + (32 * g + 8 * kk) * 2);
      qop[kk] = __builtin_bit_cast(bf16x8, u);
    }
  };

  const float c2 = a.sm_scale * kLog2e;
  bf16x8 qop[4];
  f32x4 acc[8];             // O^T tile j: acc[j][i] = o[row r][32g + 8i + j]
  float m_run = -INFINITY;  // log2 units, same in the four lanes of a row
  float l_run = 0.f;        // this lane's share of the row sum

  // Takes tile number `t` of the workgroup's stream out of the ring and
  // accumulates it; `valid` positions of the tile count.
  int cur_slot = 0, cur_h = 0;  // of the item being consumed
  auto consume_tile = [&](int t, int valid, bool is_new) -> bool {
    const int s = t % C::kSlots;
    JPT_TR(tr_t = __builtin_amdgcn_s_memrealtime();)
    if (!wait_for(&sm_filled[s], t / C::kSlots + 1)) return false;
    JPT_TR(tr_wait += __builtin_amdgcn_s_memrealtime() - tr_t; ++tr_tiles; if (!tr_first) tr_first = __builtin_amdgcn_s_memrealtime() - tr_start;)
    const char* slot = ring + s * C::kSlotBytes;
    const char* side = slot + 2 * C::kTileBytes;
    Tile<KV> tile;
    tile.read(slot, slot + C::kTileBytes, r, g, pos);
    float ks[8], vs[8], mk[8];
    if (SCALE && is_new) {
      const int64_t si = static_cast<int64_t>(cur_slot) * a.scale_heads + (a.scale_heads == 1 ? 0 : cur_h);
      const float nks = load_as_f32(a.new_k_scale, si, SCALE == kScaleF32 ? JPT_F32 : JPT_BF16);
      const float nvs = load_as_f32(a.new_v_scale, si, SCALE == kScaleF32 ? JPT_F32 : JPT_BF16);
#pragma unroll
      for (int i = 0; i < 8; ++i) { ks[i] = nks; vs[i] = nvs; }
    } else if (SCALE == kScaleF32) {
      const float* sk = reinterpret_cast<const float*>(side);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        ks[i] = sk[pos[i]];
        vs[i] = sk[32 + pos[i]];
      }
    } else if (SCALE == kScaleBF16) {
      const uint16_t* sk = reinterpret_cast<const uint16_t*>(side);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        ks[i] = bf16_bits_to_f32(sk[pos[i]]);
        vs[i] = bf16_bits_to_f32(sk[32 + pos[i]]);
      }
    }
    if (MASK) {
      const float* smk = reinterpret_cast<const float*>(side + 256);
#pragma unroll
      for (int i = 0; i < 8; ++i) mk[i] = is_new ? 0.f : smk[pos[i]];
    }
    // the registers hold the tile: hand the slot back (the release waits for
    // the LDS reads above)
    if (lane == 0)
      __hip_atomic_fetch_add(&sm_freed[s], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);

    f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tile.k_op(false, kk), qop[kk], sa, 0, 0, 0);
      sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tile.k_op(true, kk), qop[kk], sb, 0, 0, 0);
    }
    float sc[8];
    bool live[8];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float x = (i < 4 ? sa[i] : sb[i - 4]) * (SCALE ? ks[i] * c2 : c2);
      if (MASK) x += mk[i] * kLog2e;
      live[i] = pos[i] < valid && x == x;  // NaN scores attend nothing
      x = live[i] ? x : -INFINITY;
      sc[i] = x;
      tmax = fmaxf(tmax, x);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
    const float m_new = fmaxf(m_run, tmax);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_use);
    float w[8], psum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float pr = fast_exp2(sc[i] - m_use);
      psum += pr;
      w[i] = SCALE ? (live[i] ? pr * vs[i] : 0.f) : pr;
    }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] *= alpha;
    }
    const bf16x8 pop = as_op(pack_bf16(w[0], w[1]), pack_bf16(w[2], w[3]),
                             pack_bf16(w[4], w[5]), pack_bf16(w[6], w[7]));
#pragma unroll
    for (int j = 0; j < 8; ++j)
      acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tile.v_op(j), pop, acc[j], 0, 0, 0);
    return true;
  };

  // Delivers the wave's part of item number `seq` of this workgroup; the last
  // consumer to arrive folds the parts and writes the slot's output (one
  // chunk) or parks the chunk's partial (several).
  auto finish_item = [&](const Item& it, int seq) -> bool {
    const int buf = seq % C::kFoldBufs;
    // the buffer's previous item must have been folded out of it
    if (!wait_for(&sm_folded[buf], seq / C::kFoldBufs)) return false;
    float l_row = l_run + __shfl_xor(l_run, 16);
    l_row += __shfl_xor(l_row, 32);
    if (r < R) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) sm_o[buf][wave][r][o_col(32 * g + 8 * i + j)] = acc[j][i];
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
    const int64_t q_row0 = (static_cast<int64_t>(it.slot) * a.q_heads + it.h * p.rep) * a.q_rows;
    float* part = p.partials + (static_cast<int64_t>(it.part) * a.kv_heads + it.h) * R * kPartFloats;
    // four rows a pass: 16 lanes a row, eight consecutive outputs a lane
    const int d0 = 8 * (lane & 15);
    for (int row = lane >> 4; row < R; row += 4) {
      float M = -INFINITY;
#pragma unroll
      for (int w2 = 0; w2 < kConsumers; ++w2) M = fmaxf(M, sm_m[buf][w2][row]);
      float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      float l = 0.f;
#pragma unroll
      for (int w2 = 0; w2 < kConsumers; ++w2) {
        const float mw = sm_m[buf][w2][row];
        const float f = mw == -INFINITY ? 0.f : fast_exp2(mw - M);
        l += sm_l[buf][w2][row] * f;
        const float4* src = reinterpret_cast<const float4*>(&sm_o[buf][w2][row][o_col(d0)]);
        const float4 x = src[0], y = src[1];
        o[0] += x.x * f; o[1] += x.y * f; o[2] += x.z * f; o[3] += x.w * f;
        o[4] += y.x * f; o[5] += y.y * f; o[6] += y.z * f; o[7] += y.w * f;
      }
      if (it.n_chunks == 1) {
        const float inv = l > 0.f ? 1.f / l : 0.f;
        const uint4 packed = make_uint4(pack_bf16(o[0] * inv, o[1] * inv), pack_bf16(o[2] * inv, o[3] * inv),
                                        pack_bf16(o[4] * inv, o[5] * inv), pack_bf16(o[6] * inv, o[7] * inv));
        *reinterpret_cast<uint4*>(static_cast<uint16_t*>(a.out) + (q_row0 + row) * kD + d0) = packed;
        if (d0 == 0) {
          if (a.out_max) a.out_max[q_row0 + row] = M * kLn2;
          if (a.out_denom) a.out_denom[q_row0 + row] = l;
        }
      } else {
        float4* dst = reinterpret_cast<float4*>(part + row * kPartFloats + d0);
        dst[0] = make_float4(o[0], o[1], o[2], o[3]);
        dst[1] = make_float4(o[4], o[5], o[6], o[7]);
        if (d0 == 0) {
          part[row * kPartFloats + kD] = M;
          part[row * kPartFloats + kD + 1] = l;
        }
      }
    }
    if (lane == 0) {
      __hip_atomic_store(&sm_arrived[buf], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __hip_atomic_fetch_add(&sm_folded[buf], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    return true;
  };

  Item cur = fetch(0);
  if (!cur.valid) return;
  Item nxt = fetch(1);
  int base = 0;  // stream number of the current item's tile 0
  for (int k = 0;; ++k) {
    const Item nxt2 = fetch(k + 2);
    load_q(qop, cur);
    const int n_cache = cache_tiles(cur), nt = item_tiles(cur);
    cur_slot = cur.slot;
    cur_h = cur.h;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run = -INFINITY;
    l_run = 0.f;
    // this consumer's tiles: stream numbers congruent to its index
    for (int ti = (wave + kConsumers - base % kConsumers) % kConsumers; ti < nt; ti += kConsumers) {
      const bool is_new = ti >= n_cache;
      const int valid = is_new ? 1 : min(kTile, cur.count - ti * kTile);
      if (!consume_tile(base + ti, valid, is_new)) return;
    }
    JPT_TR(tr_t = __builtin_amdgcn_s_memrealtime();)
    if (!finish_item(cur, k)) return;
    JPT_TR(tr_fold += __builtin_amdgcn_s_memrealtime() - tr_t;)
    if (!nxt.valid) {
      JPT_TR(if (p.trace && lane == 0) {
        unsigned long long* o = p.trace + (static_cast<size_t>(blockIdx.x) * kWaves + wave) * 8;
        o[0] = tr_tiles; o[1] = tr_wait; o[2] = tr_fold; o[3] = __builtin_amdgcn_s_memrealtime() - tr_start;
        o[4] = tr_start; o[5] = k + 1; o[6] = tr_first; o[7] = sm_simd[hw_wave];
      })
      break;
    }
    base += nt;
    cur = nxt;
    nxt = nxt2;
  }
}

template <typename KV, bool PAGED, int SCALE, bool MASK>
void launch_rows(const FastParams& p, unsigned blocks, hipStream_t stream) {
  if (p.rows <= 4)
    hipLaunchKernelGGL((attn_decode_kernel<KV, PAGED, SCALE, MASK, 4>), dim3(blocks), dim3(kThreads), 0, stream, p);
  else if (p.rows <= 8)
    hipLaunchKernelGGL((attn_decode_kernel<KV, PAGED, SCALE, MASK, 8>), dim3(blocks), dim3(kThreads), 0, stream, p);
  else
    hipLaunchKernelGGL((attn_decode_kernel<KV, PAGED, SCALE, MASK, 16>), dim3(blocks), dim3(kThreads), 0, stream, p);
}

template <typename KV, bool PAGED, int SCALE>
void launch_masked(const FastParams& p, unsigned blocks, hipStream_t stream) {
  if (!PAGED && p.a.mask) launch_rows<KV, PAGED, SCALE, !PAGED>(p, blocks, stream);
  else launch_rows<KV, PAGED, SCALE, false>(p, blocks, stream);
}

template <typename KV>
void launch_decode(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream) {
  const int scale = !p.a.k_scale ? kNoScale : p.a.scale_dtype == JPT_F32 ? kScaleF32 : kScaleBF16;
  if (paged) {
    if (scale == kNoScale) launch_masked<KV, true, kNoScale>(p, blocks, stream);
    else if (scale == kScaleF32) launch_masked<KV, true, kScaleF32>(p, blocks, stream);
    else launch_masked<KV, true, kScaleBF16>(p, blocks, stream);
  } else {
    if (scale == kNoScale) launch_masked<KV, false, kNoScale>(p, blocks, stream);
    else if (scale == kScaleF32) launch_masked<KV, false, kScaleF32>(p, blocks, stream);
    else launch_masked<KV, false, kScaleBF16>(p, blocks, stream);
  }
}

}  // namespace decode
}  // namespace jpt
