// Ragged / dense / paged GQA decode attention for gfx950, head_dim 128.
//
// Work decomposition (split-KV).  A planning kernel turns the per-slot lengths
// into a list of chunks (slot, first position, count), longest first, sized so
// the batch yields a few work items per workgroup whatever the length
// distribution.  The attention kernel is persistent: about two 4-wavefront
// workgroups per compute unit each walk a fixed, interleaved share of the
// (chunk, KV head) items.  A wavefront streams 32-position tiles straight from
// HBM into registers (no LDS staging: every byte of K and V is needed by
// exactly one lane), converts int8 codes to bf16 in registers (exact) and runs
//     S^T = K . Q^T        v_mfma_f32_16x16x32_bf16, positions on M, the
//                          rep*q_rows query rows of the KV head on N
//     O^T = V^T . P^T      positions on the contraction index
// with an online softmax in between.  The score accumulators of lane
// (row r, group g) are exactly the probabilities that lane must feed to the
// second MFMA, so probabilities never cross lanes; the row maximum needs two
// cross-lane steps per tile.  Loads run one tile ahead of the math and the
// prefetch crosses item boundaries, so the memory pipe stays busy while an
// item is being finished (first-touch latency of a new cache row, with its
// TLB miss, is several microseconds here - longer than streaming a chunk).
// The step's own new token, when given, is one more tile of a single
// position appended to the slot's first chunk.
//
// The four waves of a workgroup are merged through LDS.  A slot that fits one
// chunk is finished in place; otherwise each chunk parks a float32 partial
// (o, max, sum) and a second small kernel folds the partials of every split
// slot.  The kernel boundary is the only device-wide synchronisation: an
// in-kernel fence costs an L2 write-back and invalidate per workgroup on this
// part and serialises per XCD.
//
// Bound: HBM bandwidth.  Algorithmic bytes per (slot, KV head) are
// len * 128 * (bytes(K) + bytes(V)) plus len * (bytes(k_scale) +
// bytes(v_scale)) / heads-sharing-a-scale; the MFMA pipes run at roughly a
// tenth of their rate at full bandwidth, the int8 -> bf16 conversion
// (1.5 VALU ops per byte) is the main issue-slot consumer.
#include <math.h>
#include <stdlib.h>

#include "attn_common.h"

namespace jpt {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kTile = 32;        // positions per wave iteration
constexpr int kD = 128;          // head_dim
constexpr int kMaxRows = 16;     // rep * q_rows
constexpr int kChunkAlign = 128;
constexpr int kItemBufs = 2;
// LDS row of 128 outputs, padded so that the 16 writers of a wave (4 rows x 4
// column groups) and the readers hit distinct banks: column d = 32g + c lives
// at 33g + c.
constexpr int kOStride = 140;
__device__ __forceinline__ int o_col(int d) { return d + (d >> 5); }
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// ---- workspace layout --------------------------------------------------------
// [0, 64 KiB)   reserved state block (kept zero)
// then          sorted plan entries, per-slot chunk table, partials
struct PlanEntry {
  int32_t slot;        // -1: unused record
  int32_t start;       // first position of the chunk
  int32_t count;       // positions in the chunk (0 for an empty slot)
  int32_t part;        // index of this chunk's partial record
  int32_t n_chunks;    // chunks of this slot
  int32_t pad[3];
};
struct SlotChunks {
  int32_t n_chunks, first_part;
};

struct Layout {
  int64_t entries, slots, partials, total;
  int32_t max_entries;
};

constexpr int kPartFloats = kD + 2;  // per row: o[128], m, l
constexpr int kMaxPlanBatch = 4096;
constexpr int kMaxChunksPerSlot = 256;

int32_t env_int(const char* name, int32_t fallback) {
  const char* e = getenv(name);
  const int32_t t = e ? atoi(e) : 0;
  return t > 0 ? t : fallback;
}

// Work items (chunk x KV head) the planner aims for.
int32_t target_items() {
  static int32_t v = env_int("JPT_ATTN_TARGET_ITEMS", 2048);
  return v;
}

int32_t persistent_blocks() {
  static int32_t v = [] {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess)
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    const int32_t per_cu = env_int("JPT_ATTN_BLOCKS_PER_CU", 2);
    return (cus * per_cu + 7) / 8 * 8;
  }();
  return v;
}

Layout make_layout(int batch, int kv_heads, int rows) {
  Layout l;
  l.max_entries = (batch + (target_items() + kv_heads - 1) / kv_heads + 1 + 7) / 8 * 8;
  auto up = [](int64_t x) { return (x + 255) / 256 * 256; };
  l.entries = JPT_ATTN_WS_STATE_BYTES;
  l.slots = up(l.entries + static_cast<int64_t>(l.max_entries) * sizeof(PlanEntry));
  l.partials = up(l.slots + static_cast<int64_t>(batch) * sizeof(SlotChunks));
  l.total = up(l.partials + static_cast<int64_t>(l.max_entries) * kv_heads * rows * kPartFloats * 4);
  return l;
}

// ---- planning kernel -----------------------------------------------------------
// One workgroup.  chunk = max(128, total positions * kv_heads / target items,
// rounded up to 128); each slot gets max(1, ceil(len / chunk)) entries
// (an empty slot still needs one item per head to write its output);
// entries are counting-sorted by tile count, longest first; records past the
// last entry are marked unused.
__global__ void __launch_bounds__(256)
plan_kernel(const int32_t* lengths, int batch, int seq_cap, int kv_heads, int target,
            PlanEntry* entries, SlotChunks* slots, int max_entries) {
  __shared__ int s_len[kMaxPlanBatch];
  __shared__ int s_first[kMaxPlanBatch];
  __shared__ long long s_total;
  __shared__ int s_chunk, s_entries;
  __shared__ int s_hist[257];
  __shared__ int s_base[257];
  const int tid = threadIdx.x;
  if (tid == 0) s_total = 0;
  for (int i = tid; i < 257; i += blockDim.x) s_hist[i] = 0;
  __syncthreads();
  long long mine = 0;
  for (int b = tid; b < batch; b += blockDim.x) {
    int n = lengths ? lengths[b] : seq_cap;
    n = n < 0 ? 0 : (n > seq_cap ? seq_cap : n);
    s_len[b] = n;
    mine += n;
  }
  atomicAdd(reinterpret_cast<unsigned long long*>(&s_total), static_cast<unsigned long long>(mine));
  __syncthreads();
  if (tid == 0) {
    long long c = (s_total * kv_heads + target - 1) / target;
    const long long floor_c = (seq_cap + kMaxChunksPerSlot - 1) / kMaxChunksPerSlot;
    c = c < floor_c ? floor_c : c;  // at most kMaxChunksPerSlot chunks per slot
    c = (c + kChunkAlign - 1) / kChunkAlign * kChunkAlign;
    s_chunk = c < kChunkAlign ? kChunkAlign : static_cast<int>(c);
    int first = 0;
    for (int b = 0; b < batch; ++b) {  // LDS only: a few cycles per slot
      s_first[b] = first;
      first += s_len[b] == 0 ? 1 : (s_len[b] + s_chunk - 1) / s_chunk;
    }
    s_entries = first;
  }
  __syncthreads();
  const int chunk = s_chunk;
  auto chunks_of = [&](int b) { return s_len[b] == 0 ? 1 : (s_len[b] + chunk - 1) / chunk; };
  auto key_of = [&](int count) {
    const int tiles = (count + kTile - 1) / kTile;
    return tiles > 256 ? 256 : tiles;
  };
  for (int b = tid; b < batch; b += blockDim.x) {
    const int nc = chunks_of(b);
    slots[b] = SlotChunks{nc, s_first[b]};
    for (int c = 0; c < nc; ++c) atomicAdd(&s_hist[key_of(min(chunk, s_len[b] - c * chunk))], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int k = 256; k >= 0; --k) {
      s_base[k] = run;
      run += s_hist[k];
    }
  }
  __syncthreads();
  for (int b = tid; b < batch; b += blockDim.x) {
    const int nc = chunks_of(b), first = s_first[b];
    for (int c = 0; c < nc; ++c) {
      const int count = min(chunk, s_len[b] - c * chunk);
      const int at = atomicAdd(&s_base[key_of(count)], 1);
      if (at < max_entries) entries[at] = PlanEntry{b, c * chunk, count, first + c, nc, {0, 0, 0}};
    }
  }
  for (int i = s_entries + tid; i < max_entries; i += blockDim.x)
    entries[i] = PlanEntry{-1, 0, 0, 0, 0, {0, 0, 0}};
}

// ---- attention kernel ------------------------------------------------------------

struct FastParams {
  jpt_attn_args a;
  const PlanEntry* entries;
  const SlotChunks* slots;
  float* partials;
  int32_t rows;  // rep * q_rows
  int32_t rep;
  int32_t total_items;  // max_entries * kv_heads
};

enum ScaleKind { kNoScale = 0, kScaleF32 = 1, kScaleBF16 = 2 };

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

template <typename KV>
struct Tile;

// int8: lane (r, g) holds bytes [32g, 32g+32) of positions r and 16+r (K) and
// bytes [8r, 8r+8) of its eight probability positions (V).
template <>
struct Tile<int8_t> {
  uint4 ka[2], kb[2];
  uint2 v[8];
  static constexpr int kElem = 1;
  __device__ __forceinline__ void load_k(const char* rowa, const char* rowb, int g) {
    const uint4* pa = reinterpret_cast<const uint4*>(rowa + 32 * g);
    const uint4* pb = reinterpret_cast<const uint4*>(rowb + 32 * g);
    ka[0] = pa[0]; ka[1] = pa[1];
    kb[0] = pb[0]; kb[1] = pb[1];
  }
  __device__ __forceinline__ void load_v(int i, const char* row, int r) {
    v[i] = *reinterpret_cast<const uint2*>(row + 8 * r);
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

// bf16: same ownership, two bytes per element.
template <>
struct Tile<__bf16> {
  uint4 ka[4], kb[4];
  uint4 v[8];
  static constexpr int kElem = 2;
  __device__ __forceinline__ void load_k(const char* rowa, const char* rowb, int g) {
    const uint4* pa = reinterpret_cast<const uint4*>(rowa + 64 * g);
    const uint4* pb = reinterpret_cast<const uint4*>(rowb + 64 * g);
#pragma unroll
    for (int i = 0; i < 4; ++i) { ka[i] = pa[i]; kb[i] = pb[i]; }
  }
  __device__ __forceinline__ void load_v(int i, const char* row, int r) {
    v[i] = *reinterpret_cast<const uint4*>(row + 16 * r);
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

// Per-position side inputs of the lane's eight score positions: two groups of
// four consecutive positions, so each is one vector load.
template <int SCALE, bool MASK>
struct Side {
  float ks[SCALE ? 8 : 1], vs[SCALE ? 8 : 1], mk[MASK ? 8 : 1];
  int valid;  // positions of the tile that are attended (tile-relative)
};

template <int SCALE>
__device__ __forceinline__ void load4_scale(float* dst, const void* base, int64_t idx) {
  if (SCALE == kScaleF32) {
    const float4 f = *reinterpret_cast<const float4*>(static_cast<const float*>(base) + idx);
    dst[0] = f.x; dst[1] = f.y; dst[2] = f.z; dst[3] = f.w;
  } else if (SCALE == kScaleBF16) {
    const uint2 u = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(base) + idx);
    dst[0] = __uint_as_float(u.x << 16); dst[1] = __uint_as_float(u.x & 0xffff0000u);
    dst[2] = __uint_as_float(u.y << 16); dst[3] = __uint_as_float(u.y & 0xffff0000u);
  }
}
template <int SCALE>
__device__ __forceinline__ float load1_scale(const void* base, int64_t idx) {
  if (SCALE == kScaleF32) return static_cast<const float*>(base)[idx];
  if (SCALE == kScaleBF16) return bf16_bits_to_f32(static_cast<const uint16_t*>(base)[idx]);
  return 1.f;
}

// One work item: a chunk of one slot for one KV head.
struct Item {
  int slot, start, count, part, n_chunks, h;
  bool valid;
};

// KV: int8_t or __bf16; PAGED: rows addressed through the page table;
// SCALE: per-position k/v scales absent, float32 or bf16; MASK: additive
// float32 mask per (slot, position).  Every tile lies inside the cache row
// (seq and page_size are multiples of 32), so loads past the chunk end stay
// in bounds; what they return is discarded by selects, never by arithmetic.
template <typename KV, bool PAGED, int SCALE, bool MASK>
__global__ void __launch_bounds__(kThreads, 2) attn_decode_kernel(FastParams p) {
  const jpt_attn_args& a = p.a;
  // Two item buffers: the waves of a workgroup never wait for one another;
  // the last wave to deliver its part of an item folds the four parts.
  __shared__ float sm_o[kItemBufs][kWaves][kMaxRows][kOStride];
  __shared__ float sm_m[kItemBufs][kWaves][kMaxRows];
  __shared__ float sm_l[kItemBufs][kWaves][kMaxRows];
  __shared__ int sm_arrived[kItemBufs];  // waves that delivered the item in this buffer
  __shared__ int sm_folded[kItemBufs];   // items folded out of this buffer so far
  if (threadIdx.x < kItemBufs) {
    sm_arrived[threadIdx.x] = 0;
    sm_folded[threadIdx.x] = 0;
  }
  __syncthreads();

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
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
      const PlanEntry en = p.entries[(m / a.kv_heads) * 8 + (i & 7)];
      it.h = m % a.kv_heads;
      it.slot = en.slot; it.start = en.start; it.count = en.count;
      it.part = en.part; it.n_chunks = en.n_chunks;
      it.valid = en.slot >= 0;
    }
    return it;
  };
  // tiles of an item: its cache positions, plus one for the new token on the
  // slot's first chunk
  auto cache_tiles = [&](const Item& it) { return (it.count + kTile - 1) / kTile; };
  auto item_tiles = [&](const Item& it) {
    return cache_tiles(it) + ((has_new && it.start == 0) ? 1 : 0);
  };

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

  constexpr int64_t kRowBytes = kD * Tile<KV>::kElem;
  const char* kbase = static_cast<const char*>(a.k);
  const char* vbase = static_cast<const char*>(a.v);
  // the lane's i-th probability position inside a tile
  auto tile_pos = [&](int i) { return 4 * g + (i & 3) + 16 * (i >> 2); };

  auto load_tile = [&](Tile<KV>& t, Side<SCALE, MASK>& s, const Item& it, int ti) {
    const int hs = a.scale_heads == 1 ? 0 : it.h;
    if (ti >= cache_tiles(it)) {
      // the new token: every row of the tile is that one token, position 0 counts
      const int64_t row = static_cast<int64_t>(it.slot) * a.kv_heads + it.h;
      const char* krow = static_cast<const char*>(a.new_k) + row * kRowBytes;
      const char* vrow = static_cast<const char*>(a.new_v) + row * kRowBytes;
      t.load_k(krow, krow, g);
#pragma unroll
      for (int i = 0; i < 8; ++i) t.load_v(i, vrow, r);
      if (SCALE) {
        const int64_t si = static_cast<int64_t>(it.slot) * a.scale_heads + hs;
        const float nks = load1_scale<SCALE>(a.new_k_scale, si);
        const float nvs = load1_scale<SCALE>(a.new_v_scale, si);
#pragma unroll
        for (int i = 0; i < 8; ++i) { s.ks[i] = nks; s.vs[i] = nvs; }
      }
      if (MASK) {
#pragma unroll
        for (int i = 0; i < 8; ++i) s.mk[i] = 0.f;
      }
      s.valid = 1;
      return;
    }
    const int t0 = it.start + ti * kTile;
    int64_t row0, srow0;  // rows of position t0
    if (PAGED) {          // a tile never straddles a page
      const int page = a.page_table[static_cast<int64_t>(it.slot) * a.max_pages + t0 / a.page_size];
      const int64_t in_pool = static_cast<int64_t>(page) * a.page_size + t0 % a.page_size;
      row0 = static_cast<int64_t>(it.h) * a.total_pages * a.page_size + in_pool;
      srow0 = static_cast<int64_t>(hs) * a.total_pages * a.page_size + in_pool;
    } else {
      row0 = (static_cast<int64_t>(it.slot) * a.kv_heads + it.h) * a.seq + t0;
      srow0 = (static_cast<int64_t>(it.slot) * a.scale_heads + hs) * a.seq + t0;
    }
    s.valid = min(kTile, it.start + it.count - t0);
    t.load_k(kbase + (row0 + r) * kRowBytes, kbase + (row0 + 16 + r) * kRowBytes, g);
    const int last = s.valid - 1;  // V rows past the chunk are re-read from its last row
#pragma unroll
    for (int i = 0; i < 8; ++i) t.load_v(i, vbase + (row0 + min(tile_pos(i), last)) * kRowBytes, r);
    if (SCALE) {
      load4_scale<SCALE>(s.ks, a.k_scale, srow0 + 4 * g);
      load4_scale<SCALE>(s.ks + 4, a.k_scale, srow0 + 16 + 4 * g);
      load4_scale<SCALE>(s.vs, a.v_scale, srow0 + 4 * g);
      load4_scale<SCALE>(s.vs + 4, a.v_scale, srow0 + 16 + 4 * g);
    }
    if (MASK) {
      const float* mrow = static_cast<const float*>(a.mask) + it.slot * a.mask_stride_b + t0;
      load4_scale<kScaleF32>(s.mk, mrow, 4 * g);
      load4_scale<kScaleF32>(s.mk + 4, mrow, 16 + 4 * g);
    }
  };

  const float c2 = a.sm_scale * kLog2e;
  bf16x8 qop[4];
  f32x4 acc[8];             // O^T tile j: acc[j][i] = o[row r][32g + 8i + j]
  float m_run = -INFINITY;  // log2 units, same in the four lanes of a row
  float l_run = 0.f;        // this lane's share of the row sum

  auto compute_tile = [&](const Tile<KV>& t, const Side<SCALE, MASK>& s) {
    f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t.k_op(false, kk), qop[kk], sa, 0, 0, 0);
      sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t.k_op(true, kk), qop[kk], sb, 0, 0, 0);
    }
    float sc[8];
    bool live[8];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float x = (i < 4 ? sa[i] : sb[i - 4]) * (SCALE ? s.ks[i] * c2 : c2);
      if (MASK) x += s.mk[i] * kLog2e;
      live[i] = tile_pos(i) < s.valid && x == x;  // NaN scores attend nothing
      x = live[i] ? x : -INFINITY;
      sc[i] = x;
      tmax = fmaxf(tmax, x);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
    const float m_new = fmaxf(m_run, tmax);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = exp2f(m_run - m_use);
    float w[8], psum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float pr = exp2f(sc[i] - m_use);
      psum += pr;
      w[i] = SCALE ? (live[i] ? pr * s.vs[i] : 0.f) : pr;
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
      acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t.v_op(j), pop, acc[j], 0, 0, 0);
  };

  // Finishes the wave's part of item number `seq` of this workgroup: deliver
  // (o, max, sum) to the item's LDS buffer; the last wave to arrive folds the
  // four parts and writes the slot's output (one chunk) or parks the chunk's
  // partial (several).  No workgroup barrier: the other waves go on streaming.
  auto finish_item = [&](const Item& it, int seq) {
    const int buf = seq % kItemBufs;
    // the buffer's previous item (seq - kItemBufs) must have been folded; a
    // wave would have to run two whole items ahead of a sibling to wait here
    while (__hip_atomic_load(&sm_folded[buf], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < seq / kItemBufs)
      __builtin_amdgcn_s_sleep(1);
    float l_row = l_run + __shfl_xor(l_run, 16);
    l_row += __shfl_xor(l_row, 32);
    if (r < R) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) sm_o[buf][wave][r][33 * g + 8 * i + j] = acc[j][i];
      if (g == 0) {
        sm_m[buf][wave][r] = m_run;
        sm_l[buf][wave][r] = l_row;
      }
    }
    int arrived = 0;
    if (lane == 0)
      arrived = __hip_atomic_fetch_add(&sm_arrived[buf], 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
    arrived = __builtin_amdgcn_readfirstlane(arrived);
    if (arrived != kWaves - 1) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    const int64_t q_row0 = (static_cast<int64_t>(it.slot) * a.q_heads + it.h * p.rep) * a.q_rows;
    float* part = p.partials + (static_cast<int64_t>(it.part) * a.kv_heads + it.h) * R * kPartFloats;
    for (int idx = lane; idx < R * kD; idx += 64) {
      const int row = idx / kD, d = idx % kD;
      float M = -INFINITY;
#pragma unroll
      for (int w2 = 0; w2 < kWaves; ++w2) M = fmaxf(M, sm_m[buf][w2][row]);
      float o = 0.f, l = 0.f;
#pragma unroll
      for (int w2 = 0; w2 < kWaves; ++w2) {
        const float mw = sm_m[buf][w2][row];
        const float f = mw == -INFINITY ? 0.f : exp2f(mw - M);
        o += sm_o[buf][w2][row][o_col(d)] * f;
        l += sm_l[buf][w2][row] * f;
      }
      if (it.n_chunks == 1) {
        static_cast<uint16_t*>(a.out)[(q_row0 + row) * kD + d] = f32_to_bf16_bits(l > 0.f ? o / l : 0.f);
        if (d == 0) {
          if (a.out_max) a.out_max[q_row0 + row] = M * kLn2;
          if (a.out_denom) a.out_denom[q_row0 + row] = l;
        }
      } else {
        part[row * kPartFloats + d] = o;
        if (d == 0) {
          part[row * kPartFloats + kD] = M;
          part[row * kPartFloats + kD + 1] = l;
        }
      }
    }
    if (lane == 0) {
      __hip_atomic_store(&sm_arrived[buf], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __hip_atomic_fetch_add(&sm_folded[buf], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  };

  Item cur = fetch(0);
  if (!cur.valid) return;
  Item nxt = fetch(1);
  load_q(qop, cur);
  Tile<KV> ta, tb;
  Side<SCALE, MASK> sa_, sb_;
  bool in_b = false;  // which buffer holds the wave's current tile
  if (wave < item_tiles(cur)) load_tile(ta, sa_, cur, wave);

  for (int k = 0;; ++k) {
    const Item nxt2 = fetch(k + 2);  // entries are read two items ahead of their use
    bf16x8 qn[4];
    if (nxt.valid) load_q(qn, nxt);
    const int nt_cur = item_tiles(cur);
    const int nt_nxt = nxt.valid ? item_tiles(nxt) : 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run = -INFINITY;
    l_run = 0.f;

    int ti = wave;
    if (ti >= nt_cur && wave < nt_nxt) {  // nothing to do here: start on the next item's first tile
      if (in_b) load_tile(tb, sb_, nxt, wave);
      else load_tile(ta, sa_, nxt, wave);
    }
    while (ti < nt_cur) {
      const int tn = ti + kWaves;
      // the tile after this one: same item, or the first tile of the next item
      if (in_b) {
        if (tn < nt_cur) load_tile(ta, sa_, cur, tn);
        else if (wave < nt_nxt) load_tile(ta, sa_, nxt, wave);
        compute_tile(tb, sb_);
      } else {
        if (tn < nt_cur) load_tile(tb, sb_, cur, tn);
        else if (wave < nt_nxt) load_tile(tb, sb_, nxt, wave);
        compute_tile(ta, sa_);
      }
      in_b = !in_b;
      ti = tn;
    }
    finish_item(cur, k);
    if (!nxt.valid) break;
    cur = nxt;
    nxt = nxt2;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) qop[kk] = qn[kk];
  }
}

// Folds the partials of every slot that was split into several chunks: one
// workgroup per (slot, KV head).  The chunk maxima and sums go through LDS
// first; then thread (row, d) walks the chunks with independent loads, eight
// in flight.
__global__ void __launch_bounds__(512) attn_merge_kernel(FastParams p) {
  const jpt_attn_args& a = p.a;
  const int b = blockIdx.x / a.kv_heads, h = blockIdx.x % a.kv_heads;
  const SlotChunks sc = p.slots[b];
  if (sc.n_chunks <= 1) return;
  __shared__ float s_mc[kMaxChunksPerSlot * kMaxRows];  // [chunk][row]
  __shared__ float s_lc[kMaxChunksPerSlot * kMaxRows];
  __shared__ float s_m[kMaxRows], s_l[kMaxRows];
  const int R = p.rows, n = sc.n_chunks;
  const int tid = threadIdx.x;
  const int64_t rec = static_cast<int64_t>(R) * kPartFloats;
  const float* first = p.partials + (static_cast<int64_t>(sc.first_part) * a.kv_heads + h) * rec;
  const int64_t step = static_cast<int64_t>(a.kv_heads) * rec;
  const int64_t q_row0 = (static_cast<int64_t>(b) * a.q_heads + h * p.rep) * a.q_rows;
  for (int i = tid; i < n * R; i += blockDim.x) {
    const float* base = first + (i / R) * step + (i % R) * kPartFloats;
    s_mc[i] = base[kD];
    s_lc[i] = base[kD + 1];
  }
  __syncthreads();
  if (tid < R) {
    float M = -INFINITY, L = 0.f;
    for (int c = 0; c < n; ++c) M = fmaxf(M, s_mc[c * R + tid]);
    for (int c = 0; c < n; ++c) {
      const float mc = s_mc[c * R + tid];
      L += mc == -INFINITY ? 0.f : exp2f(mc - M) * s_lc[c * R + tid];
    }
    s_m[tid] = M;
    s_l[tid] = L;
  }
  __syncthreads();
  for (int idx = tid; idx < R * kD; idx += blockDim.x) {
    const int row = idx / kD, d = idx % kD;
    const float M = s_m[row], L = s_l[row];
    const float* col = first + row * kPartFloats + d;
    float o = 0.f;
#pragma unroll 8
    for (int c = 0; c < n; ++c) {
      const float mc = s_mc[c * R + row];
      o += col[c * step] * (mc == -INFINITY ? 0.f : exp2f(mc - M));
    }
    static_cast<uint16_t*>(a.out)[(q_row0 + row) * kD + d] = f32_to_bf16_bits(L > 0.f ? o / L : 0.f);
    if (d == 0) {
      if (a.out_max) a.out_max[q_row0 + row] = M * kLn2;
      if (a.out_denom) a.out_denom[q_row0 + row] = L;
    }
  }
}

template <typename KV, bool PAGED, int SCALE>
void launch_masked(const FastParams& p, unsigned blocks, hipStream_t stream) {
  if (!PAGED && p.a.mask)
    hipLaunchKernelGGL((attn_decode_kernel<KV, PAGED, SCALE, !PAGED>), dim3(blocks), dim3(kThreads), 0, stream, p);
  else
    hipLaunchKernelGGL((attn_decode_kernel<KV, PAGED, SCALE, false>), dim3(blocks), dim3(kThreads), 0, stream, p);
}

template <typename KV, bool PAGED>
void launch_scaled(const FastParams& p, unsigned blocks, hipStream_t stream) {
  if (!p.a.k_scale) launch_masked<KV, PAGED, kNoScale>(p, blocks, stream);
  else if (p.a.scale_dtype == JPT_F32) launch_masked<KV, PAGED, kScaleF32>(p, blocks, stream);
  else launch_masked<KV, PAGED, kScaleBF16>(p, blocks, stream);
}

}  // namespace

bool attn_fast_supported(const jpt_attn_args& a, AttnMode mode) {
  if (a.force_generic) return false;
  if (a.dim != kD || a.q_dtype != JPT_BF16) return false;
  if (a.kv_dtype != JPT_I8 && a.kv_dtype != JPT_BF16) return false;
  const int rows = a.q_heads / a.kv_heads * a.q_rows;
  if (rows > kMaxRows) return false;
  if (a.batch > kMaxPlanBatch) return false;
  // tiles of 32 positions must stay inside a cache row / a page
  if (mode == kPaged ? a.page_size % kTile != 0 : a.seq % kTile != 0) return false;
  if (a.mask && (a.mask_stride_h != 0 || a.q_rows != 1 || a.mask_dtype != JPT_F32 ||
                 a.mask_stride_b % 4 != 0 || !aligned(a.mask, 16)))
    return false;
  if (a.k_scale && (!aligned(a.k_scale, 16) || !aligned(a.v_scale, 16))) return false;
  if (!aligned(a.q, 16) || !aligned(a.k, 16) || !aligned(a.v, 16)) return false;
  if (a.new_k && (!aligned(a.new_k, 16) || !aligned(a.new_v, 16))) return false;
  return true;
}

int64_t attn_fast_workspace_bytes(const jpt_attn_args& a) {
  const int rows = a.q_heads / a.kv_heads * a.q_rows;
  return make_layout(a.batch, a.kv_heads, rows).total;
}

int32_t attn_plan_launch(const jpt_attn_args& a, bool paged, hipStream_t stream) {
  const int rows = a.q_heads / a.kv_heads * a.q_rows;
  const Layout l = make_layout(a.batch, a.kv_heads, rows);
  JPT_REQUIRE(a.workspace != nullptr && a.workspace_bytes >= l.total,
              "workspace of %lld bytes needed, %lld given", static_cast<long long>(l.total),
              static_cast<long long>(a.workspace_bytes));
  JPT_REQUIRE(aligned(a.workspace, 256), "workspace must be 256-byte aligned");
  JPT_REQUIRE(a.batch <= kMaxPlanBatch, "batch above %d", kMaxPlanBatch);
  char* ws = static_cast<char*>(a.workspace);
  const int cap = paged ? a.max_pages * a.page_size : a.seq;
  JPT_REQUIRE(cap > 0, "sequence capacity must be positive");
  hipLaunchKernelGGL(plan_kernel, dim3(1), dim3(256), 0, stream, a.lengths, a.batch, cap,
                     a.kv_heads, target_items(), reinterpret_cast<PlanEntry*>(ws + l.entries),
                     reinterpret_cast<SlotChunks*>(ws + l.slots), l.max_entries);
  return launch_status("plan_kernel");
}

int32_t attn_fast_launch(const jpt_attn_args& a, AttnMode mode, hipStream_t stream) {
  const int rep = a.q_heads / a.kv_heads;
  const int rows = rep * a.q_rows;
  const Layout l = make_layout(a.batch, a.kv_heads, rows);
  JPT_REQUIRE(a.workspace != nullptr && a.workspace_bytes >= l.total,
              "workspace of %lld bytes needed, %lld given", static_cast<long long>(l.total),
              static_cast<long long>(a.workspace_bytes));
  JPT_REQUIRE(aligned(a.workspace, 256), "workspace must be 256-byte aligned");
  char* ws = static_cast<char*>(a.workspace);
  FastParams p{};
  p.a = a;
  p.entries = reinterpret_cast<const PlanEntry*>(ws + l.entries);
  p.slots = reinterpret_cast<const SlotChunks*>(ws + l.slots);
  p.partials = reinterpret_cast<float*>(ws + l.partials);
  p.rows = rows;
  p.rep = rep;
  p.total_items = l.max_entries * a.kv_heads;
  if (!a.reuse_plan) {
    int32_t st = attn_plan_launch(a, mode == kPaged, stream);
    if (st != JPT_OK) return st;
  }
  int32_t blocks = persistent_blocks();
  if (blocks > p.total_items) blocks = p.total_items;  // total_items is a multiple of 8
  const bool paged = mode == kPaged;
  if (a.kv_dtype == JPT_I8) {
    if (paged) launch_scaled<int8_t, true>(p, blocks, stream);
    else launch_scaled<int8_t, false>(p, blocks, stream);
  } else {
    if (paged) launch_scaled<__bf16, true>(p, blocks, stream);
    else launch_scaled<__bf16, false>(p, blocks, stream);
  }
  int32_t st = launch_status("attn_decode_kernel");
  if (st != JPT_OK) return st;
  hipLaunchKernelGGL(attn_merge_kernel, dim3(a.batch * a.kv_heads), dim3(512), 0, stream, p);
  return launch_status("attn_merge_kernel");
}

}  // namespace jpt

extern "C" {

int64_t jpt_attn_workspace_bytes(const jpt_attn_args* args) {
  if (args == nullptr || args->batch <= 0 || args->kv_heads <= 0 || args->q_heads <= 0 ||
      args->q_rows <= 0)
    return JPT_ATTN_WS_STATE_BYTES;
  return jpt::attn_fast_workspace_bytes(*args);
}

static int32_t attn_entry(const jpt_attn_args* args, jpt::AttnMode mode, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(args != nullptr, "args is NULL");
  int32_t st = check_attn_args(*args, mode);
  if (st != JPT_OK) return st;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (attn_fast_supported(*args, mode)) return attn_fast_launch(*args, mode, s);
  return attn_generic_launch(*args, mode, s);
}

int32_t jpt_attn_plan(const jpt_attn_args* args, int32_t paged, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(args != nullptr, "args is NULL");
  JPT_REQUIRE(args->batch > 0 && args->kv_heads > 0 && args->q_heads > 0 && args->q_rows > 0 &&
                  args->q_heads % args->kv_heads == 0, "batch, heads and q_rows must be positive");
  return attn_plan_launch(*args, paged != 0, static_cast<hipStream_t>(stream));
}

int32_t jpt_attn_ragged(const jpt_attn_args* args, void* stream) { return attn_entry(args, jpt::kRagged, stream); }
int32_t jpt_attn_dense(const jpt_attn_args* args, void* stream) { return attn_entry(args, jpt::kDense, stream); }
int32_t jpt_attn_paged(const jpt_attn_args* args, void* stream) { return attn_entry(args, jpt::kPaged, stream); }

}  // extern "C"
