// Ragged / dense / paged GQA decode attention for gfx950, head_dim 128.
//
// Work decomposition (split-KV): a small planning kernel turns the per-slot
// lengths into a list of (slot, first position, count) chunks, sized so that
// the whole batch yields a few thousand workgroups whatever the length
// distribution, longest chunks first.  The attention kernel runs one
// 4-wavefront workgroup per (chunk, KV head); wave w streams the 32-position
// tiles w, w+4, ... of the chunk straight from HBM into registers (no LDS
// staging: every byte of K and V is needed by exactly one lane), converts
// int8 codes to bf16 in registers (exact) and runs
//     S^T = K . Q^T        v_mfma_f32_16x16x32_bf16, positions on M, the
//                          rep*q_rows query rows of the KV head on N
//     O^T = V^T . P^T      positions on the contraction index
// with an online softmax in between.  The score accumulators of lane
// (row r, group g) are exactly the probabilities that lane must feed to the
// second MFMA, so probabilities never cross lanes; the row maximum needs two
// cross-lane steps per tile.  Waves are merged through LDS, chunks of one
// (slot, head) through a float32 partial buffer: the last workgroup to arrive
// (device-scope counter) folds the partials, adds the optional new-token term
// and writes the output, so there is no separate merge launch.
//
// Bound: HBM bandwidth.  Algorithmic bytes per (slot, KV head) are
// len * 128 * (bytes(K) + bytes(V)) plus len * (bytes(k_scale) +
// bytes(v_scale)) / heads-sharing-a-scale; the MFMA pipes run at roughly a
// tenth of their rate at full bandwidth, the int8 -> bf16 conversion
// (1.5 VALU ops per byte) is the main issue-slot consumer.
#include <math.h>

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
constexpr int kChunkAlign = kTile * kWaves;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// ---- workspace layout --------------------------------------------------------
// [0, 64 KiB)   arrival counters, one int32 per (slot, KV head); zero between calls
// then          PlanHeader, sorted entries, per-slot chunk tables, partials
struct PlanHeader {
  int32_t n_entries;
  int32_t chunk;
  int32_t pad[2];
};
struct PlanEntry {
  int32_t slot, start, count, part;  // part: index of this chunk's partial record
};

struct Layout {
  int64_t header, entries, slot_first, slot_nchunks, partials, total;
  int32_t max_entries;
};

constexpr int kPartFloats = kD + 2;  // per row: o[128], m, l

int32_t default_target_items() {
  static int32_t v = [] {
    const char* e = getenv("JPT_ATTN_TARGET_ITEMS");
    int32_t t = e ? atoi(e) : 0;
    return t > 0 ? t : 2048;
  }();
  return v;
}

Layout make_layout(int batch, int kv_heads, int rows) {
  Layout l;
  const int target = default_target_items();
  l.max_entries = batch + (target + kv_heads - 1) / kv_heads + 1;
  auto up = [](int64_t x) { return (x + 255) / 256 * 256; };
  l.header = JPT_ATTN_WS_STATE_BYTES;
  l.entries = l.header + 256;
  l.slot_first = up(l.entries + static_cast<int64_t>(l.max_entries) * sizeof(PlanEntry));
  l.slot_nchunks = up(l.slot_first + static_cast<int64_t>(batch) * 4);
  l.partials = up(l.slot_nchunks + static_cast<int64_t>(batch) * 4);
  l.total = up(l.partials + static_cast<int64_t>(l.max_entries) * kv_heads * rows * kPartFloats * 4);
  return l;
}

// ---- planning kernel -----------------------------------------------------------
// One workgroup.  chunk = max(128, total positions * kv_heads / target items,
// rounded up to 128); each slot gets max(1, ceil(len / chunk)) entries
// (an empty slot still needs one workgroup per head to write its zeros);
// entries are counting-sorted by tile count, longest first.
__global__ void __launch_bounds__(256)
plan_kernel(const int32_t* lengths, int batch, int seq_cap, int kv_heads, int target_items,
            PlanHeader* header, PlanEntry* entries, int32_t* slot_first, int32_t* slot_nchunks,
            int max_entries) {
  __shared__ long long s_total;
  __shared__ int s_chunk;
  __shared__ int s_hist[257];
  __shared__ int s_base[257];
  const int tid = threadIdx.x;
  if (tid == 0) s_total = 0;
  for (int i = tid; i < 257; i += blockDim.x) s_hist[i] = 0;
  __syncthreads();
  auto len_of = [&](int b) {
    int n = lengths ? lengths[b] : seq_cap;
    return n < 0 ? 0 : (n > seq_cap ? seq_cap : n);
  };
  long long mine = 0;
  for (int b = tid; b < batch; b += blockDim.x) mine += len_of(b);
  atomicAdd(reinterpret_cast<unsigned long long*>(&s_total), static_cast<unsigned long long>(mine));
  __syncthreads();
  if (tid == 0) {
    long long c = (s_total * kv_heads + target_items - 1) / target_items;
    c = (c + kChunkAlign - 1) / kChunkAlign * kChunkAlign;
    s_chunk = c < kChunkAlign ? kChunkAlign : static_cast<int>(c);
    int first = 0;
    for (int b = 0; b < batch; ++b) {  // batch is a few hundred at most
      const int n = len_of(b);
      const int nc = n == 0 ? 1 : (n + s_chunk - 1) / s_chunk;
      slot_first[b] = first;
      slot_nchunks[b] = nc;
      first += nc;
    }
    header->n_entries = first < max_entries ? first : max_entries;
    header->chunk = s_chunk;
  }
  __syncthreads();
  const int chunk = s_chunk;
  auto key_of = [&](int count) {
    const int tiles = (count + kTile - 1) / kTile;
    return tiles > 256 ? 256 : tiles;
  };
  for (int b = tid; b < batch; b += blockDim.x) {
    const int n = len_of(b), nc = slot_nchunks[b];
    for (int c = 0; c < nc; ++c) atomicAdd(&s_hist[key_of(min(chunk, n - c * chunk))], 1);
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
    const int n = len_of(b), nc = slot_nchunks[b], first = slot_first[b];
    for (int c = 0; c < nc; ++c) {
      const int count = min(chunk, n - c * chunk);
      const int at = atomicAdd(&s_base[key_of(count)], 1);
      if (at < max_entries) entries[at] = PlanEntry{b, c * chunk, count, first + c};
    }
  }
}

// ---- attention kernel ------------------------------------------------------------

struct FastParams {
  jpt_attn_args a;
  const PlanHeader* header;
  const PlanEntry* entries;
  const int32_t* slot_first;
  const int32_t* slot_nchunks;
  float* partials;
  int32_t* counters;
  int32_t rows;  // rep * q_rows
  int32_t rep;
};

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

// Per-position side inputs of the lane's eight score positions.
struct Side {
  float ks[8], vs[8], mk[8];
};

template <typename KV, bool PAGED>
__global__ void __launch_bounds__(kThreads, 2) attn_decode_kernel(FastParams p) {
  const jpt_attn_args& a = p.a;
  __shared__ float sm_o[kWaves][kMaxRows][kD];
  __shared__ float sm_m[kWaves][kMaxRows];
  __shared__ float sm_l[kWaves][kMaxRows];
  __shared__ float blk_m[kMaxRows], blk_l[kMaxRows];
  __shared__ float sm_new[kMaxRows];
  __shared__ int sm_last;

  // block -> (entry, head): all heads of an entry share an
  // XCD (block ids go round-robin over the 8 XCDs), so its scales and page
  // table row are fetched into one L2 only.
  const int xcd = blockIdx.x & 7, j_in_xcd = blockIdx.x >> 3;
  const int e = (j_in_xcd / a.kv_heads) * 8 + xcd;
  const int h = j_in_xcd % a.kv_heads;
  if (e >= p.header->n_entries) return;
  const PlanEntry ent = p.entries[e];
  const int b = ent.slot;
  const int n_chunks = p.slot_nchunks[b];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int R = p.rows;
  const int hs = a.scale_heads == 1 ? 0 : h;

  // Q^T operand: lane (r, g) holds q[row r][32g + 8kk + i], zero for r >= R
  bf16x8 qop[4];
  {
    const char* qrow = static_cast<const char*>(a.q) +
                       ((static_cast<int64_t>(b) * a.q_heads + h * p.rep) * a.q_rows + r) * (kD * 2);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      uint4 u = make_uint4(0, 0, 0, 0);
      if (r < R) u = *reinterpret_cast<const uint4*>(qrow + (32 * g + 8 * kk) * 2);
      qop[kk] = __builtin_bit_cast(bf16x8, u);
    }
  }

  const int chunk_end = ent.start + ent.count;  // first position not attended here
  const int n_tiles = (ent.count + kTile - 1) / kTile;
  const float c2 = a.sm_scale * kLog2e;
  const bool has_scale = a.k_scale != nullptr;
  const bool has_mask = a.mask != nullptr;
  constexpr int64_t kRowBytes = kD * Tile<KV>::kElem;

  // byte address of the K/V row of position `tok` (clamped to a live one)
  auto row_offset = [&](int tok) -> int64_t {
    tok = min(tok, chunk_end - 1);
    if (PAGED) {
      const int page = a.page_table[static_cast<int64_t>(b) * a.max_pages + tok / a.page_size];
      return ((static_cast<int64_t>(h) * a.total_pages + page) * a.page_size + tok % a.page_size) * kRowBytes;
    }
    return ((static_cast<int64_t>(b) * a.kv_heads + h) * a.seq + tok) * kRowBytes;
  };
  auto scale_index = [&](int tok) -> int64_t {
    tok = min(tok, chunk_end - 1);
    if (PAGED) {
      const int page = a.page_table[static_cast<int64_t>(b) * a.max_pages + tok / a.page_size];
      return (static_cast<int64_t>(hs) * a.total_pages + page) * a.page_size + tok % a.page_size;
    }
    return (static_cast<int64_t>(b) * a.scale_heads + hs) * a.seq + tok;
  };
  // the lane's i-th probability position inside a tile
  auto tile_pos = [&](int i) { return 4 * g + (i & 3) + 16 * (i >> 2); };

  auto load_tile = [&](Tile<KV>& t, Side& s, int ti) {
    const int t0 = ent.start + ti * kTile;
    const char* kbase = static_cast<const char*>(a.k);
    const char* vbase = static_cast<const char*>(a.v);
    t.load_k(kbase + row_offset(t0 + r), kbase + row_offset(t0 + 16 + r), g);
#pragma unroll
    for (int i = 0; i < 8; ++i) t.load_v(i, vbase + row_offset(t0 + tile_pos(i)), r);
    if (has_scale) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int64_t si = scale_index(t0 + tile_pos(i));
        s.ks[i] = load_as_f32(a.k_scale, si, a.scale_dtype);
        s.vs[i] = load_as_f32(a.v_scale, si, a.scale_dtype);
      }
    }
    if (has_mask) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int tok = min(t0 + tile_pos(i), chunk_end - 1);
        s.mk[i] = load_as_f32(a.mask, b * a.mask_stride_b + tok, a.mask_dtype);
      }
    }
  };

  f32x4 acc[8];  // O^T tile j: acc[j][i] = o[row r][32g + 8i + j]
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY;  // log2 units, same in the four lanes of a row
  float l_run = 0.f;        // this lane's share of the row sum

  auto compute_tile = [&](const Tile<KV>& t, const Side& s, int ti) {
    const int t0 = ent.start + ti * kTile;
    f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t.k_op(false, kk), qop[kk], sa, 0, 0, 0);
      sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t.k_op(true, kk), qop[kk], sb, 0, 0, 0);
    }
    float sc[8];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float x = (i < 4 ? sa[i] : sb[i - 4]) * (has_scale ? s.ks[i] * c2 : c2);
      if (has_mask) x += s.mk[i] * kLog2e;
      if (t0 + tile_pos(i) >= chunk_end) x = -INFINITY;
      if (x != x) x = -INFINITY;  // NaN scores (e.g. -inf mask on garbage) attend nothing
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
      w[i] = has_scale ? pr * s.vs[i] : pr;
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

  // software pipeline: the next tile's loads are in flight during this tile's math
  {
    Tile<KV> t0, t1;
    Side s0, s1;
    int ti = wave;
    if (ti < n_tiles) load_tile(t0, s0, ti);
    while (ti < n_tiles) {
      if (ti + kWaves < n_tiles) load_tile(t1, s1, ti + kWaves);
      compute_tile(t0, s0, ti);
      ti += kWaves;
      if (ti >= n_tiles) break;
      if (ti + kWaves < n_tiles) load_tile(t0, s0, ti + kWaves);
      compute_tile(t1, s1, ti);
      ti += kWaves;
    }
  }

  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);

  // ---- merge the four waves through LDS ----
  if (r < R) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) sm_o[wave][r][32 * g + 8 * i + j] = acc[j][i];
    if (g == 0) {
      sm_m[wave][r] = m_run;
      sm_l[wave][r] = l_run;
    }
  }
  __syncthreads();
  // block result: o in sm_o[0] (each element is read and rewritten by one
  // thread only), max and sum in blk_m / blk_l
  for (int idx = tid; idx < R * kD; idx += kThreads) {
    const int row = idx / kD, d = idx % kD;
    float M = -INFINITY;
#pragma unroll
    for (int w2 = 0; w2 < kWaves; ++w2) M = fmaxf(M, sm_m[w2][row]);
    float o = 0.f, l = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < kWaves; ++w2) {
      const float mw = sm_m[w2][row];
      const float f = mw == -INFINITY ? 0.f : exp2f(mw - M);
      o += sm_o[w2][row][d] * f;
      l += sm_l[w2][row] * f;
    }
    sm_o[0][row][d] = o;
    if (d == 0) {
      blk_m[row] = M;
      blk_l[row] = l;
    }
  }
  __syncthreads();

  // ---- several chunks: park the partial, the last arrival folds them all ----
  if (n_chunks > 1) {
    const int64_t rec = static_cast<int64_t>(R) * kPartFloats;  // floats per (chunk, head)
    float* mine = p.partials + (static_cast<int64_t>(ent.part) * a.kv_heads + h) * rec;
    for (int idx = tid; idx < R * kD; idx += kThreads)
      mine[(idx / kD) * kPartFloats + idx % kD] = sm_o[0][idx / kD][idx % kD];
    if (tid < R) {
      mine[tid * kPartFloats + kD] = blk_m[tid];
      mine[tid * kPartFloats + kD + 1] = blk_l[tid];
    }
    __threadfence();  // partial visible device-wide before the arrival is counted
    __syncthreads();
    if (tid == 0) {
      int32_t* counter = p.counters + b * a.kv_heads + h;
      const int arrived = atomicAdd(counter, 1);
      sm_last = arrived == n_chunks - 1;
      if (sm_last) *counter = 0;  // everyone has arrived: leave it zero for the next call
    }
    __syncthreads();
    if (!sm_last) return;
    __threadfence();
    const float* first = p.partials + (static_cast<int64_t>(p.slot_first[b]) * a.kv_heads + h) * rec;
    const int64_t step = static_cast<int64_t>(a.kv_heads) * rec;
    for (int idx = tid; idx < R * kD; idx += kThreads) {
      const int row = idx / kD, d = idx % kD;
      float M = -INFINITY;
      for (int c = 0; c < n_chunks; ++c) M = fmaxf(M, first[c * step + row * kPartFloats + kD]);
      float o = 0.f, l = 0.f;
      for (int c = 0; c < n_chunks; ++c) {
        const float* pc = first + c * step + row * kPartFloats;
        const float f = pc[kD] == -INFINITY ? 0.f : exp2f(pc[kD] - M);
        o += pc[d] * f;
        l += pc[kD + 1] * f;
      }
      sm_o[0][row][d] = o;
      if (d == 0) {
        blk_m[row] = M;
        blk_l[row] = l;
      }
    }
    __syncthreads();
  }

  // ---- the step's own token: one more position, merged by log-sum-exp ----
  const int64_t q_row0 = (static_cast<int64_t>(b) * a.q_heads + h * p.rep) * a.q_rows;
  const int64_t new_row = static_cast<int64_t>(b) * a.kv_heads + h;
  float new_vs = 1.f;
  if (a.new_k) {
    float new_ks = 1.f;
    if (a.new_k_scale) {
      new_ks = load_as_f32(a.new_k_scale, static_cast<int64_t>(b) * a.scale_heads + hs, a.scale_dtype);
      new_vs = load_as_f32(a.new_v_scale, static_cast<int64_t>(b) * a.scale_heads + hs, a.scale_dtype);
    }
    if (wave == 0) {
      const float k0 = load_as_f32(a.new_k, new_row * kD + 2 * lane, a.kv_dtype);
      const float k1 = load_as_f32(a.new_k, new_row * kD + 2 * lane + 1, a.kv_dtype);
      for (int row = 0; row < R; ++row) {
        float part = load_as_f32(a.q, (q_row0 + row) * kD + 2 * lane, JPT_BF16) * k0 +
                     load_as_f32(a.q, (q_row0 + row) * kD + 2 * lane + 1, JPT_BF16) * k1;
        for (int off = 32; off > 0; off >>= 1) part += __shfl_xor(part, off);
        if (lane == 0) sm_new[row] = part * c2 * new_ks;
      }
    }
    __syncthreads();
  }

  // ---- output ----
  for (int idx = tid; idx < R * kD; idx += kThreads) {
    const int row = idx / kD, d = idx % kD;
    float M = blk_m[row], L = blk_l[row], o = sm_o[0][row][d];
    if (a.new_k) {
      const float s = sm_new[row];
      const float M2 = fmaxf(M, s);
      const float fa = M == -INFINITY ? 0.f : exp2f(M - M2);
      const float fb = exp2f(s - M2);
      o = o * fa + fb * new_vs * load_as_f32(a.new_v, new_row * kD + d, a.kv_dtype);
      L = L * fa + fb;
      M = M2;
    }
    static_cast<uint16_t*>(a.out)[(q_row0 + row) * kD + d] = f32_to_bf16_bits(L > 0.f ? o / L : 0.f);
    if (d == 0) {
      if (a.out_max) a.out_max[q_row0 + row] = M * kLn2;
      if (a.out_denom) a.out_denom[q_row0 + row] = L;
    }
  }
}

template <typename KV, bool PAGED>
void launch_decode(const FastParams& p, unsigned blocks, hipStream_t stream) {
  hipLaunchKernelGGL((attn_decode_kernel<KV, PAGED>), dim3(blocks), dim3(kThreads), 0, stream, p);
}

}  // namespace

bool attn_fast_supported(const jpt_attn_args& a, AttnMode mode) {
  if (a.force_generic) return false;
  if (a.dim != kD || a.q_dtype != JPT_BF16) return false;
  if (a.kv_dtype != JPT_I8 && a.kv_dtype != JPT_BF16) return false;
  const int rows = a.q_heads / a.kv_heads * a.q_rows;
  if (rows > kMaxRows) return false;
  if (static_cast<int64_t>(a.batch) * a.kv_heads * 4 > JPT_ATTN_WS_STATE_BYTES) return false;
  if (mode == kPaged && a.page_size % kTile != 0) return false;
  if (a.mask && (a.mask_stride_h != 0 || a.q_rows != 1)) return false;
  if (!aligned(a.q, 16) || !aligned(a.k, 16) || !aligned(a.v, 16)) return false;
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
  char* ws = static_cast<char*>(a.workspace);
  const int cap = paged ? a.max_pages * a.page_size : a.seq;
  JPT_REQUIRE(cap > 0, "sequence capacity must be positive");
  hipLaunchKernelGGL(plan_kernel, dim3(1), dim3(256), 0, stream, a.lengths, a.batch, cap,
                     a.kv_heads, default_target_items(),
                     reinterpret_cast<PlanHeader*>(ws + l.header),
                     reinterpret_cast<PlanEntry*>(ws + l.entries),
                     reinterpret_cast<int32_t*>(ws + l.slot_first),
                     reinterpret_cast<int32_t*>(ws + l.slot_nchunks), l.max_entries);
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
  p.header = reinterpret_cast<const PlanHeader*>(ws + l.header);
  p.entries = reinterpret_cast<const PlanEntry*>(ws + l.entries);
  p.slot_first = reinterpret_cast<const int32_t*>(ws + l.slot_first);
  p.slot_nchunks = reinterpret_cast<const int32_t*>(ws + l.slot_nchunks);
  p.partials = reinterpret_cast<float*>(ws + l.partials);
  p.counters = reinterpret_cast<int32_t*>(ws);
  p.rows = rows;
  p.rep = rep;
  if (!a.reuse_plan) {
    int32_t st = attn_plan_launch(a, mode == kPaged, stream);
    if (st != JPT_OK) return st;
  }
  const unsigned blocks = static_cast<unsigned>((l.max_entries + 7) / 8 * 8) * a.kv_heads;
  const bool paged = mode == kPaged;
  if (a.kv_dtype == JPT_I8) {
    if (paged) launch_decode<int8_t, true>(p, blocks, stream);
    else launch_decode<int8_t, false>(p, blocks, stream);
  } else {
    if (paged) launch_decode<__bf16, true>(p, blocks, stream);
    else launch_decode<__bf16, false>(p, blocks, stream);
  }
  return launch_status("attn_decode_kernel");
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
  JPT_REQUIRE(static_cast<int64_t>(args->batch) * args->kv_heads * 4 <= JPT_ATTN_WS_STATE_BYTES,
              "batch * kv_heads too large for the planned kernel");
  return attn_plan_launch(*args, paged != 0, static_cast<hipStream_t>(stream));
}

int32_t jpt_attn_ragged(const jpt_attn_args* args, void* stream) { return attn_entry(args, jpt::kRagged, stream); }
int32_t jpt_attn_dense(const jpt_attn_args* args, void* stream) { return attn_entry(args, jpt::kDense, stream); }
int32_t jpt_attn_paged(const jpt_attn_args* args, void* stream) { return attn_entry(args, jpt::kPaged, stream); }

}  // extern "C"
