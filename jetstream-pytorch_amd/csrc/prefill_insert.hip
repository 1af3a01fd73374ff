// Prefill -> decode insert: a prompt's K and V rows (heads, tokens, dim) written
// into one slot of a dense cache (with ring wrap) or into the slot's pages,
// either copied or quantised per token to int8 with the insert quantiser.
//
// One workgroup per (token, K|V).  HBM-bound data movement: reads the prompt
// once (the quantising pass re-reads it from cache), writes codes and scales.
#include "common.h"

namespace jpt {
namespace {

// Layers that are tensors of their own (no common stride) come as a table of
// pointers inside the kernel arguments.
constexpr int kTableLayers = 64;
struct InsertParams {
  jpt_prefill_insert_args a;
  int32_t use_table;
  const void* src_k[kTableLayers];
  const void* src_v[kTableLayers];
  void* dst_k[kTableLayers];
  void* dst_v[kTableLayers];
  void* k_scale[kTableLayers];
  void* v_scale[kTableLayers];
};

// Source, destination and scale tensor of (layer, K|V): the table's, or the
// first layer's moved on by the layer strides.
__device__ __forceinline__ void layer_tensors(const InsertParams& p, int layer, bool is_v, int esz_in, int esz_out,
                                              int esz_scale, const void** src, char** dst, void** scale) {
  const jpt_prefill_insert_args& a = p.a;
  if (p.use_table) {
    *src = is_v ? p.src_v[layer] : p.src_k[layer];
    *dst = static_cast<char*>(is_v ? p.dst_v[layer] : p.dst_k[layer]);
    *scale = is_v ? p.v_scale[layer] : p.k_scale[layer];
    return;
  }
  *src = static_cast<const char*>(is_v ? a.src_v : a.src_k) + layer * a.src_layer_stride * esz_in;
  *dst = static_cast<char*>(is_v ? a.dst_v : a.dst_k) + layer * a.dst_layer_stride * esz_out;
  void* s0 = is_v ? a.v_scale : a.k_scale;
  *scale = s0 == nullptr ? nullptr : static_cast<char*>(s0) + layer * a.scale_layer_stride * esz_scale;
}

template <bool ROUND_BF16>
__device__ __forceinline__ float rnd(float x) {
  return ROUND_BF16 ? round_to_bf16(x) : x;
}

// four consecutive elements of the source row as float
__device__ __forceinline__ void load4(const void* src, int64_t i, int dtype, float* x) {
  if (dtype == JPT_BF16) {
    const uint2 raw = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(src) + i);
    x[0] = __uint_as_float(raw.x << 16);
    x[1] = __uint_as_float(raw.x & 0xffff0000u);
    x[2] = __uint_as_float(raw.y << 16);
    x[3] = __uint_as_float(raw.y & 0xffff0000u);
  } else {
    const float4 raw = *reinterpret_cast<const float4*>(static_cast<const float*>(src) + i);
    x[0] = raw.x; x[1] = raw.y; x[2] = raw.z; x[3] = raw.w;
  }
}

// dim % 4 == 0.  The op order of the quantiser is that of
// jpt_kv_append_quant_i8 (each op rounded to the scale dtype):
//   trunc: a = absmax; s = a / 127;             q = x / s;      code = trunc(q)
//   rne:   a = max(absmax, eps); s = a / 127; r = 1 / s; q = x * r;
//          code = clamp(rint(q), -128, 127)
template <bool BF16_MATH>
__global__ void __launch_bounds__(256) prefill_insert_kernel(InsertParams p) {
  const jpt_prefill_insert_args& a = p.a;
  const int t = blockIdx.x;
  const bool is_v = blockIdx.y == 1;
  const int layer = blockIdx.z;
  const bool paged = a.page_ids != nullptr;
  const bool quant = a.dst_dtype == JPT_I8 && a.in_dtype != JPT_I8;
  const int H = a.heads, D = a.dim, HD = H * D;
  const int esz_in = a.in_dtype == JPT_F32 ? 4 : a.in_dtype == JPT_BF16 ? 2 : 1;
  const int esz_out = quant ? 1 : esz_in;
  const int esz_scale = a.scale_dtype == JPT_F32 ? 4 : 2;
  const void* src;
  char* dst;
  void* scale_out;
  layer_tensors(p, layer, is_v, esz_in, esz_out, esz_scale, &src, &dst, &scale_out);

  // destination row of (this token, head h): element index row * D
  int64_t pool_row = 0;  // dense: position in the slot's row; paged: row in the pool
  if (paged) {
    const int page = a.page_ids[t / a.page_size];
    if (page < 0 || page >= a.total_pages) return;
    pool_row = static_cast<int64_t>(page) * a.page_size + t % a.page_size;
  } else {
    int at = (a.start + t) % a.seq;
    pool_row = at < 0 ? at + a.seq : at;
  }
  auto row_of = [&](int h) -> int64_t {
    return paged ? static_cast<int64_t>(h) * a.total_pages * a.page_size + pool_row
                 : (static_cast<int64_t>(a.slot) * H + h) * a.seq + pool_row;
  };
  auto scale_index = [&](int g) -> int64_t {
    return paged ? static_cast<int64_t>(g) * a.total_pages * a.page_size + pool_row
                 : (static_cast<int64_t>(a.slot) * a.scale_heads + g) * a.seq + pool_row;
  };

  if (t >= a.tokens) {  // paged only: the tail of the last page is zero-filled
    for (int i = 4 * threadIdx.x; i < HD; i += 4 * blockDim.x) {
      const int h = i / D, d = i - h * D;
      char* out = dst + (row_of(h) * D + d) * esz_out;
      if (esz_out == 1) *reinterpret_cast<uint32_t*>(out) = 0u;
      else if (esz_out == 2) *reinterpret_cast<uint2*>(out) = make_uint2(0u, 0u);
      else *reinterpret_cast<uint4*>(out) = make_uint4(0u, 0u, 0u, 0u);
    }
    return;
  }
  const int64_t head_stride = a.src_head_stride > 0 ? a.src_head_stride : static_cast<int64_t>(a.tokens) * D;
  auto src_index = [&](int h, int d) -> int64_t { return h * head_stride + static_cast<int64_t>(t) * D + d; };

  if (!quant) {  // copy
    for (int i = 4 * threadIdx.x; i < HD; i += 4 * blockDim.x) {
      const int h = i / D, d = i - h * D;
      const char* in = static_cast<const char*>(src) + src_index(h, d) * esz_in;
      char* out = dst + (row_of(h) * D + d) * esz_in;
      if (esz_in == 1) *reinterpret_cast<uint32_t*>(out) = *reinterpret_cast<const uint32_t*>(in);
      else if (esz_in == 2) *reinterpret_cast<uint2*>(out) = *reinterpret_cast<const uint2*>(in);
      else *reinterpret_cast<uint4*>(out) = *reinterpret_cast<const uint4*>(in);
    }
    return;
  }

  __shared__ float s_red[4];
  __shared__ float s_scale[64];
  const int groups = a.scale_heads;  // 1 or H
  const int per_group = HD / groups;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int g = 0; g < groups; ++g) {
    float m = 0.f;
    for (int i = 4 * threadIdx.x; i < per_group; i += 4 * blockDim.x) {
      const int e = g * per_group + i, h = e / D, d = e - h * D;
      float x[4];
      load4(src, src_index(h, d), a.in_dtype, x);
      m = fmaxf(m, fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3]))));
    }
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if (lane == 0) s_red[wave] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
      float amax = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
      if (a.rounding == JPT_ROUND_RNE) amax = fmaxf(amax, rnd<BF16_MATH>(1e-5f));
      s_scale[g] = rnd<BF16_MATH>(amax / 127.0f);
    }
    __syncthreads();
  }
  for (int i = 4 * threadIdx.x; i < HD; i += 4 * blockDim.x) {
    const int h = i / D, d = i - h * D;
    const float s = s_scale[groups == 1 ? 0 : h];
    float x[4];
    load4(src, src_index(h, d), a.in_dtype, x);
    int code[4];
    if (a.rounding == JPT_ROUND_TRUNC) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float q = rnd<BF16_MATH>(x[j] / s);
        code[j] = (q != q) ? 0 : static_cast<int>(q);
      }
    } else {
      const float r = rnd<BF16_MATH>(1.0f / s);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float q = rnd<BF16_MATH>(x[j] * r);
        code[j] = static_cast<int>(fminf(fmaxf(rintf(q), -128.f), 127.f));
      }
    }
    const uint32_t packed = (static_cast<uint32_t>(code[0]) & 0xffu) | ((static_cast<uint32_t>(code[1]) & 0xffu) << 8) |
                            ((static_cast<uint32_t>(code[2]) & 0xffu) << 16) | (static_cast<uint32_t>(code[3]) << 24);
    *reinterpret_cast<uint32_t*>(dst + row_of(h) * D + d) = packed;
  }
  if (threadIdx.x < groups) store_from_f32(scale_out, scale_index(threadIdx.x), a.scale_dtype, s_scale[threadIdx.x]);
}

// The common quantising shape - bf16 prompt, heads * dim == 1024 - eight tokens
// a workgroup, two at a time: 128 threads a token, each keeping its eight
// elements (one 16-byte load) of four tokens in registers between the absmax
// pass and the quantise pass, so the prompt is read once, in wide loads that
// are all issued before the first wait.  Same op order as the general kernel.
constexpr int kTokensPerBlock = 8;
// Tokens t0 .. t0 + 7 of the prompt `a` describes (tokens, page_ids, n_pages,
// src_head_stride), read from src, written to dst / scale_out.
template <bool BF16_MATH>
__device__ __forceinline__ void quant_insert_tokens(const jpt_prefill_insert_args& a, const uint16_t* src, char* dst,
                                                    void* scale_out, int t0) {
  constexpr int kPasses = kTokensPerBlock / 2;
  const int half = threadIdx.x >> 7;  // which of the pass's two tokens
  const bool paged = a.page_ids != nullptr;
  const int H = a.heads, D = a.dim;
  const int rows = paged ? a.n_pages * a.page_size : a.tokens;
  const int i0 = 8 * (threadIdx.x & 127), h = i0 / D, d = i0 - h * D;
  const int groups = a.scale_heads;
  const int64_t head_stride = a.src_head_stride > 0 ? a.src_head_stride : static_cast<int64_t>(a.tokens) * D;

  // every load of the workgroup before anything waits for one (addresses
  // clamped into the prompt, results masked afterwards); page ids likewise
  uint4 raw[kPasses];
#pragma unroll
  for (int j = 0; j < kPasses; ++j) {
    const int t = min(t0 + 2 * j + half, a.tokens - 1);
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 w = __builtin_nontemporal_load(
        reinterpret_cast<const u32x4*>(src + h * head_stride + static_cast<int64_t>(t) * D + d));  // read once
    raw[j] = make_uint4(w.x, w.y, w.z, w.w);
  }
  int page_of[kPasses];
#pragma unroll
  for (int j = 0; j < kPasses; ++j)
    page_of[j] = paged ? a.page_ids[min(t0 + 2 * j + half, rows - 1) / a.page_size] : 0;
  float x[kPasses][8], m[kPasses];
  int64_t pool_row[kPasses];  // dense: position in the slot's row; paged: row in the pool; -1: nothing to write
#pragma unroll
  for (int j = 0; j < kPasses; ++j) {
    const int t = t0 + 2 * j + half;
    pool_row[j] = -1;
    if (t < rows) {
      if (paged) {
        const int page = page_of[j];
        if (page >= 0 && page < a.total_pages) pool_row[j] = static_cast<int64_t>(page) * a.page_size + t % a.page_size;
      } else {
        const int at = (a.start + t) % a.seq;
        pool_row[j] = at < 0 ? at + a.seq : at;
      }
    }
    const bool live = t < a.tokens;
    const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
    m[j] = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[j][2 * i] = live ? __uint_as_float(w[i] << 16) : 0.f;
      x[j][2 * i + 1] = live ? __uint_as_float(w[i] & 0xffff0000u) : 0.f;
      m[j] = fmaxf(m[j], fmaxf(fabsf(x[j][2 * i]), fabsf(x[j][2 * i + 1])));
    }
  }
  __shared__ float s_red[kPasses][4];
  if (groups == 1) {
#pragma unroll
    for (int j = 0; j < kPasses; ++j) {
      for (int off = 32; off > 0; off >>= 1) m[j] = fmaxf(m[j], __shfl_xor(m[j], off));
      if ((threadIdx.x & 63) == 0) s_red[j][threadIdx.x >> 6] = m[j];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kPasses; ++j) m[j] = fmaxf(s_red[j][2 * half], s_red[j][2 * half + 1]);
  } else {
    // a head's D / 8 threads are consecutive; D / 8 is a power of two <= 64
#pragma unroll
    for (int j = 0; j < kPasses; ++j)
      for (int off = D / 16; off > 0; off >>= 1) m[j] = fmaxf(m[j], __shfl_xor(m[j], off));
  }
#pragma unroll
  for (int j = 0; j < kPasses; ++j) {
    if (pool_row[j] < 0) continue;
    const int64_t row = paged ? static_cast<int64_t>(h) * a.total_pages * a.page_size + pool_row[j]
                              : (static_cast<int64_t>(a.slot) * H + h) * a.seq + pool_row[j];
    uint2* out = reinterpret_cast<uint2*>(dst + row * D + d);
    if (t0 + 2 * j + half >= a.tokens) {  // paged only: the tail of the last page is zero-filled
      *out = make_uint2(0u, 0u);
      continue;
    }
    float amax = m[j];
    if (a.rounding == JPT_ROUND_RNE) amax = fmaxf(amax, rnd<BF16_MATH>(1e-5f));
    const float s = rnd<BF16_MATH>(amax / 127.0f);
    uint32_t code[8];
    if (a.rounding == JPT_ROUND_TRUNC) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float q = rnd<BF16_MATH>(x[j][i] / s);
        code[i] = static_cast<uint32_t>((q != q) ? 0 : static_cast<int>(q)) & 0xffu;
      }
    } else {
      const float r = rnd<BF16_MATH>(1.0f / s);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float q = rnd<BF16_MATH>(x[j][i] * r);
        code[i] = static_cast<uint32_t>(static_cast<int>(fminf(fmaxf(rintf(q), -128.f), 127.f))) & 0xffu;
      }
    }
    // written once, read by later launches only: keep it out of the way of the prompt being read
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 packed = {code[0] | (code[1] << 8) | (code[2] << 16) | (code[3] << 24),
                          code[4] | (code[5] << 8) | (code[6] << 16) | (code[7] << 24)};
    __builtin_nontemporal_store(packed, reinterpret_cast<u32x2*>(out));
    if (groups == 1 ? (threadIdx.x & 127) == 0 : d == 0) {
      const int g = groups == 1 ? 0 : h;
      const int64_t idx = paged ? static_cast<int64_t>(g) * a.total_pages * a.page_size + pool_row[j]
                                : (static_cast<int64_t>(a.slot) * groups + g) * a.seq + pool_row[j];
      store_from_f32(scale_out, idx, a.scale_dtype, s);
    }
  }
}

// The same for the Llama shape, 8 heads of 128 elements, laid out for memory: a
// thread keeps one 16-byte piece of one token's row in four heads (passes), so
// that the 64 lanes of a wave read four consecutive tokens' rows of one head -
// 1 KiB in one piece - and write 512 contiguous bytes of codes, where the
// mapping above touches four heads' 256 bytes.  A token's absmax: over the
// thread's four heads, the 16 lanes that share the token, and (one scale a
// token) the workgroup's other half, which has the other four heads.
template <bool BF16_MATH>
__device__ __forceinline__ void quant_insert_tokens_8x128(const jpt_prefill_insert_args& a, const uint16_t* src, char* dst,
                                                          void* scale_out, int t0) {
  constexpr int H = 8, D = 128, kHeadsPerThread = 4;
  const int piece = threadIdx.x & 15, tq = (threadIdx.x >> 4) & 7, hg = threadIdx.x >> 7;
  const bool paged = a.page_ids != nullptr;
  const int rows = paged ? a.n_pages * a.page_size : a.tokens;
  const int groups = a.scale_heads;
  const int64_t head_stride = a.src_head_stride > 0 ? a.src_head_stride : static_cast<int64_t>(a.tokens) * D;
  const int t = t0 + tq, d = 8 * piece;
  const int t_src = min(t, a.tokens - 1);
  uint4 raw[kHeadsPerThread];
#pragma unroll
  for (int j = 0; j < kHeadsPerThread; ++j) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 w = __builtin_nontemporal_load(
        reinterpret_cast<const u32x4*>(src + (hg * kHeadsPerThread + j) * head_stride + static_cast<int64_t>(t_src) * D + d));
    raw[j] = make_uint4(w.x, w.y, w.z, w.w);
  }
  const int page = paged ? a.page_ids[min(t, rows - 1) / a.page_size] : 0;
  int64_t pool_row = -1;  // dense: position in the slot's row; paged: row in the pool; -1: nothing to write
  if (t < rows) {
    if (paged) {
      if (page >= 0 && page < a.total_pages) pool_row = static_cast<int64_t>(page) * a.page_size + t % a.page_size;
    } else {
      const int at = (a.start + t) % a.seq;
      pool_row = at < 0 ? at + a.seq : at;
    }
  }
  const bool live = t < a.tokens;
  float x[kHeadsPerThread][8], m[kHeadsPerThread];
#pragma unroll
  for (int j = 0; j < kHeadsPerThread; ++j) {
    const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
    m[j] = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[j][2 * i] = live ? __uint_as_float(w[i] << 16) : 0.f;
      x[j][2 * i + 1] = live ? __uint_as_float(w[i] & 0xffff0000u) : 0.f;
      m[j] = fmaxf(m[j], fmaxf(fabsf(x[j][2 * i]), fabsf(x[j][2 * i + 1])));
    }
    for (int off = 8; off > 0; off >>= 1) m[j] = fmaxf(m[j], __shfl_xor(m[j], off));  // the head's 16 pieces
  }
  __shared__ float s_half[2][kTokensPerBlock];
  if (groups == 1) {
    const float mine = fmaxf(fmaxf(m[0], m[1]), fmaxf(m[2], m[3]));
    if (piece == 0) s_half[hg][tq] = mine;
    __syncthreads();
    const float all = fmaxf(s_half[0][tq], s_half[1][tq]);
#pragma unroll
    for (int j = 0; j < kHeadsPerThread; ++j) m[j] = all;
  }
  if (pool_row < 0) return;
#pragma unroll
  for (int j = 0; j < kHeadsPerThread; ++j) {
    const int h = hg * kHeadsPerThread + j;
    const int64_t row = paged ? static_cast<int64_t>(h) * a.total_pages * a.page_size + pool_row
                              : (static_cast<int64_t>(a.slot) * H + h) * a.seq + pool_row;
    uint2* out = reinterpret_cast<uint2*>(dst + row * D + d);
    if (!live) {  // paged only: the tail of the last page is zero-filled
      *out = make_uint2(0u, 0u);
      continue;
    }
    float amax = m[j];
    if (a.rounding == JPT_ROUND_RNE) amax = fmaxf(amax, rnd<BF16_MATH>(1e-5f));
    const float s = rnd<BF16_MATH>(amax / 127.0f);
    uint32_t code[8];
    if (a.rounding == JPT_ROUND_TRUNC) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float q = rnd<BF16_MATH>(x[j][i] / s);
        code[i] = static_cast<uint32_t>((q != q) ? 0 : static_cast<int>(q)) & 0xffu;
      }
    } else {
      const float r = rnd<BF16_MATH>(1.0f / s);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float q = rnd<BF16_MATH>(x[j][i] * r);
        code[i] = static_cast<uint32_t>(static_cast<int>(fminf(fmaxf(rintf(q), -128.f), 127.f))) & 0xffu;
      }
    }
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 packed = {code[0] | (code[1] << 8) | (code[2] << 16) | (code[3] << 24),
                          code[4] | (code[5] << 8) | (code[6] << 16) | (code[7] << 24)};
    __builtin_nontemporal_store(packed, reinterpret_cast<u32x2*>(out));
    if (piece == 0 && (groups == 1 ? (hg == 0 && j == 0) : true)) {
      const int g = groups == 1 ? 0 : h;
      const int64_t idx = paged ? static_cast<int64_t>(g) * a.total_pages * a.page_size + pool_row
                                : (static_cast<int64_t>(a.slot) * groups + g) * a.seq + pool_row;
      store_from_f32(scale_out, idx, a.scale_dtype, s);
    }
  }
}

template <bool BF16_MATH>
__global__ void __launch_bounds__(256) prefill_insert_quant4_kernel(InsertParams p) {
  const jpt_prefill_insert_args& a = p.a;
  const bool is_v = blockIdx.y == 1;
  const void* src;
  char* dst;
  void* scale_out;
  layer_tensors(p, blockIdx.z, is_v, 2, 1, a.scale_dtype == JPT_F32 ? 4 : 2, &src, &dst, &scale_out);
  if (a.heads == 8 && a.dim == 128)
    quant_insert_tokens_8x128<BF16_MATH>(a, static_cast<const uint16_t*>(src), dst, scale_out, blockIdx.x * kTokensPerBlock);
  else
    quant_insert_tokens<BF16_MATH>(a, static_cast<const uint16_t*>(src), dst, scale_out, blockIdx.x * kTokensPerBlock);
}

// Several prompts into the pages of one stacked pool in one launch: the
// workgroups of all prompts side by side (prompt r owns those from
// first_block[r] on), layers along z by the layer strides.
constexpr int kLaunchPrompts = 32;
struct PromptsParams {
  jpt_prefill_insert_args a;  // destination, geometry, dtypes; its source and page fields are unused
  int32_t n_prompts;
  int32_t first_block[kLaunchPrompts + 1];
  jpt_insert_prompt prompt[kLaunchPrompts];
};

template <bool BF16_MATH>
__global__ void __launch_bounds__(256) prefill_insert_prompts_kernel(PromptsParams p) {
  int r = 0;
  while (r + 1 < p.n_prompts && static_cast<int>(blockIdx.x) >= p.first_block[r + 1]) ++r;
  const jpt_insert_prompt& pr = p.prompt[r];
  jpt_prefill_insert_args a = p.a;
  a.tokens = pr.tokens;
  a.n_pages = pr.n_pages;
  a.page_ids = pr.page_ids;
  a.src_head_stride = pr.src_head_stride;
  const bool is_v = blockIdx.y == 1;
  const int layer = blockIdx.z;
  const uint16_t* src = static_cast<const uint16_t*>(is_v ? pr.src_v : pr.src_k) + layer * pr.src_layer_stride;
  char* dst = static_cast<char*>(is_v ? a.dst_v : a.dst_k) + layer * a.dst_layer_stride;
  const int esz_scale = a.scale_dtype == JPT_F32 ? 4 : 2;
  void* scale_out = static_cast<char*>(is_v ? a.v_scale : a.k_scale) + layer * a.scale_layer_stride * esz_scale;
  const int t0 = (static_cast<int>(blockIdx.x) - p.first_block[r]) * kTokensPerBlock;
  if (a.heads == 8 && a.dim == 128) quant_insert_tokens_8x128<BF16_MATH>(a, src, dst, scale_out, t0);
  else quant_insert_tokens<BF16_MATH>(a, src, dst, scale_out, t0);
}

}  // namespace
}  // namespace jpt

namespace jpt {
namespace {

// Checks and launches.  layers == nullptr: the tensors of args, n_layers of them
// a layer stride apart; else a table of at most kTableLayers layers.
int32_t insert_launch(const jpt_prefill_insert_args& a, const jpt_insert_layer* layers, int32_t n_table, void* stream) {
  JPT_REQUIRE(a.tokens >= 0 && a.heads > 0 && a.dim > 0, "tokens, heads, dim out of range");
  JPT_REQUIRE(a.dim % 4 == 0, "dim must be a multiple of 4");
  JPT_REQUIRE(a.in_dtype == JPT_BF16 || a.in_dtype == JPT_F32 || a.in_dtype == JPT_I8, "bad in_dtype");
  const bool quant = a.dst_dtype == JPT_I8 && a.in_dtype != JPT_I8;
  JPT_REQUIRE(quant || a.dst_dtype == a.in_dtype, "dst_dtype must be in_dtype (copy) or int8 (quantise)");
  const int esz = a.in_dtype == JPT_F32 ? 4 : a.in_dtype == JPT_BF16 ? 2 : 1;
  const int esz_out = quant ? 1 : esz;
  JPT_REQUIRE(a.src_head_stride == 0 || (a.src_head_stride >= static_cast<int64_t>(a.tokens) * a.dim && a.src_head_stride % 4 == 0),
              "src_head_stride must cover the tokens and be a multiple of 4");
  if (quant) {
    JPT_REQUIRE(a.scale_dtype == a.in_dtype || a.scale_dtype == JPT_F32, "scale_dtype must equal in_dtype or be f32");
    JPT_REQUIRE(a.scale_heads == 1 || a.scale_heads == a.heads, "scale_heads must be 1 or heads");
    JPT_REQUIRE(a.scale_heads <= 64, "per-head scales support at most 64 heads");
    JPT_REQUIRE(a.rounding == JPT_ROUND_TRUNC || a.rounding == JPT_ROUND_RNE, "bad rounding mode");
  }
  InsertParams p{};
  p.a = a;
  bool wide_ok = true;  // every tensor is aligned for the wide quantising kernel
  auto check_layer = [&](const void* sk, const void* sv, const void* dk, const void* dv, const void* ks,
                         const void* vs) -> int32_t {
    JPT_REQUIRE(sk && sv && dk && dv, "NULL tensor argument");
    JPT_REQUIRE(aligned(sk, 4 * esz) && aligned(sv, 4 * esz), "source rows must be aligned to four elements");
    JPT_REQUIRE(aligned(dk, 4 * esz_out) && aligned(dv, 4 * esz_out), "destination must be aligned to four elements");
    if (quant) JPT_REQUIRE(ks && vs, "k_scale/v_scale are NULL");
    wide_ok = wide_ok && aligned(sk, 16) && aligned(sv, 16) && aligned(dk, 8) && aligned(dv, 8);
    return JPT_OK;
  };
  if (layers) {
    JPT_REQUIRE(n_table >= 1 && n_table <= kTableLayers, "1..%d layers a table", kTableLayers);
    p.use_table = 1;
    p.a.n_layers = n_table;
    for (int l = 0; l < n_table; ++l) {
      const jpt_insert_layer& t = layers[l];
      const int32_t st = check_layer(t.src_k, t.src_v, t.dst_k, t.dst_v, t.k_scale, t.v_scale);
      if (st != JPT_OK) return st;
      p.src_k[l] = t.src_k; p.src_v[l] = t.src_v;
      p.dst_k[l] = t.dst_k; p.dst_v[l] = t.dst_v;
      p.k_scale[l] = t.k_scale; p.v_scale[l] = t.v_scale;
    }
  } else {
    const int32_t st = check_layer(a.src_k, a.src_v, a.dst_k, a.dst_v, a.k_scale, a.v_scale);
    if (st != JPT_OK) return st;
    JPT_REQUIRE(a.src_layer_stride % 4 == 0 && a.dst_layer_stride % 4 == 0, "layer strides must be multiples of 4");
    if (p.a.n_layers <= 0) p.a.n_layers = 1;
    JPT_REQUIRE(p.a.n_layers <= 65535, "n_layers out of range");
    wide_ok = wide_ok && a.src_layer_stride % 8 == 0 && a.dst_layer_stride % 8 == 0;
  }
  int32_t rows = a.tokens;
  if (a.page_ids) {
    JPT_REQUIRE(a.total_pages > 0 && a.page_size > 0 && a.n_pages >= 0, "paged geometry out of range");
    JPT_REQUIRE(static_cast<int64_t>(a.n_pages) * a.page_size >= a.tokens, "too few pages for %d tokens", a.tokens);
    rows = a.n_pages * a.page_size;
  } else {
    JPT_REQUIRE(a.seq > 0 && a.batch > 0 && a.slot >= 0 && a.slot < a.batch, "slot or seq out of range");
    JPT_REQUIRE(a.tokens <= a.seq, "%d tokens do not fit a cache of %d positions", a.tokens, a.seq);
  }
  if (rows == 0) return JPT_OK;
  const int d8 = a.dim / 8;  // threads a head in the wide kernel
  const bool four = quant && wide_ok && a.tokens > 0 && a.in_dtype == JPT_BF16 && a.heads * a.dim == 1024 &&
                    a.dim % 8 == 0 && (a.scale_heads == 1 || (d8 <= 64 && (d8 & (d8 - 1)) == 0)) &&
                    (a.src_head_stride == 0 || a.src_head_stride % 8 == 0);
  if (four) {
    dim3 grid4((rows + kTokensPerBlock - 1) / kTokensPerBlock, 2, p.a.n_layers);
    if (a.scale_dtype == JPT_BF16)
      hipLaunchKernelGGL(prefill_insert_quant4_kernel<true>, grid4, dim3(256), 0, static_cast<hipStream_t>(stream), p);
    else
      hipLaunchKernelGGL(prefill_insert_quant4_kernel<false>, grid4, dim3(256), 0, static_cast<hipStream_t>(stream), p);
    return launch_status("prefill_insert_quant4_kernel");
  }
  dim3 grid(rows, 2, p.a.n_layers);
  if (quant && a.scale_dtype == JPT_BF16)
    hipLaunchKernelGGL(prefill_insert_kernel<true>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), p);
  else
    hipLaunchKernelGGL(prefill_insert_kernel<false>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), p);
  return launch_status("prefill_insert_kernel");
}

}  // namespace
}  // namespace jpt

extern "C" {

int32_t jpt_prefill_insert(const jpt_prefill_insert_args* args, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(args != nullptr, "args is NULL");
  return insert_launch(*args, nullptr, 0, stream);
}

int32_t jpt_prefill_insert_layers(const jpt_prefill_insert_args* args, const jpt_insert_layer* layers,
                                  int32_t n_layers, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(args != nullptr && layers != nullptr, "NULL argument");
  JPT_REQUIRE(n_layers >= 1, "n_layers must be positive");
  for (int32_t l0 = 0; l0 < n_layers; l0 += kTableLayers) {
    const int32_t n = n_layers - l0 < kTableLayers ? n_layers - l0 : kTableLayers;
    const int32_t st = insert_launch(*args, layers + l0, n, stream);
    if (st != JPT_OK) return st;
  }
  return JPT_OK;
}

int32_t jpt_prefill_insert_prompts(const jpt_prefill_insert_args* args, const jpt_insert_prompt* prompts,
                                   int32_t n_prompts, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(args != nullptr && prompts != nullptr, "NULL argument");
  JPT_REQUIRE(n_prompts >= 1, "n_prompts must be positive");
  const jpt_prefill_insert_args& a = *args;
  const int n_layers = a.n_layers > 0 ? a.n_layers : 1;
  const int d8 = a.dim / 8;
  // the shape the one-launch kernel takes; anything else goes prompt by prompt
  bool wide = a.dst_dtype == JPT_I8 && a.in_dtype == JPT_BF16 && a.heads * a.dim == 1024 && a.dim % 8 == 0 &&
              a.heads > 0 && (a.scale_heads == 1 || (a.scale_heads == a.heads && d8 <= 64 && (d8 & (d8 - 1)) == 0)) &&
              a.dst_k && a.dst_v && a.k_scale && a.v_scale && aligned(a.dst_k, 8) && aligned(a.dst_v, 8) &&
              a.dst_layer_stride % 8 == 0 && a.total_pages > 0 && a.page_size > 0 && n_layers <= 65535 &&
              (a.scale_dtype == JPT_BF16 || a.scale_dtype == JPT_F32) &&
              (a.rounding == JPT_ROUND_TRUNC || a.rounding == JPT_ROUND_RNE);
  for (int32_t r = 0; r < n_prompts && wide; ++r) {
    const jpt_insert_prompt& pr = prompts[r];
    wide = pr.src_k && pr.src_v && pr.page_ids && pr.tokens > 0 && pr.n_pages > 0 &&
           static_cast<int64_t>(pr.n_pages) * a.page_size >= pr.tokens && aligned(pr.src_k, 16) &&
           aligned(pr.src_v, 16) && pr.src_layer_stride % 8 == 0 &&
           (pr.src_head_stride == 0 || (pr.src_head_stride % 8 == 0 &&
                                        pr.src_head_stride >= static_cast<int64_t>(pr.tokens) * a.dim));
  }
  if (!wide) {
    for (int32_t r = 0; r < n_prompts; ++r) {
      jpt_prefill_insert_args one = a;
      one.src_k = prompts[r].src_k;
      one.src_v = prompts[r].src_v;
      one.page_ids = prompts[r].page_ids;
      one.tokens = prompts[r].tokens;
      one.n_pages = prompts[r].n_pages;
      one.src_head_stride = prompts[r].src_head_stride;
      one.src_layer_stride = prompts[r].src_layer_stride;
      const int32_t st = insert_launch(one, nullptr, 0, stream);
      if (st != JPT_OK) return st;
    }
    return JPT_OK;
  }
  for (int32_t r0 = 0; r0 < n_prompts; r0 += kLaunchPrompts) {
    PromptsParams p{};
    p.a = a;
    p.a.n_layers = n_layers;
    p.n_prompts = n_prompts - r0 < kLaunchPrompts ? n_prompts - r0 : kLaunchPrompts;
    int blocks = 0;
    for (int r = 0; r < p.n_prompts; ++r) {
      p.prompt[r] = prompts[r0 + r];
      p.first_block[r] = blocks;
      blocks += (prompts[r0 + r].n_pages * a.page_size + kTokensPerBlock - 1) / kTokensPerBlock;
    }
    p.first_block[p.n_prompts] = blocks;
    const dim3 grid(blocks, 2, n_layers);
    if (a.scale_dtype == JPT_BF16)
      hipLaunchKernelGGL(prefill_insert_prompts_kernel<true>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), p);
    else
      hipLaunchKernelGGL(prefill_insert_prompts_kernel<false>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), p);
    const int32_t st = launch_status("prefill_insert_prompts_kernel");
    if (st != JPT_OK) return st;
  }
  return JPT_OK;
}

}  // extern "C"
