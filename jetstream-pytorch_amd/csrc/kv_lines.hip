// Per-slot KV line writes: plain scatter (bf16/f32/int8 caches and scalers,
// one or all layers) and the fused per-token absmax int8 quantiser + scatter.
//
// Both are pure data movement bound by HBM bandwidth and, at decode sizes
// (one token per slot), by launch latency: one launch covers K and V (and
// both scalers) for every layer.
#include "common.h"

namespace jpt {
namespace {

struct LineParams {
  jpt_line_tensor t[JPT_MAX_LINE_TENSORS];
  int32_t vec[JPT_MAX_LINE_TENSORS];  // bytes one thread moves, per tensor
  const int32_t* pos;
  int32_t pos_count, n_layers, batch, seq;
};

template <typename V>
__device__ __forceinline__ void copy_vec(void* dst, const void* src, int v) {
  static_cast<V*>(dst)[v] = static_cast<const V*>(src)[v];
}

// grid.y = tensor; a thread moves one vector of one (layer, slot, head) line.
__global__ void __launch_bounds__(256) scatter_lines_kernel(LineParams p) {
  const jpt_line_tensor t = p.t[blockIdx.y];
  const int vec = p.vec[blockIdx.y];
  const int vec_per_row = t.row_bytes / vec;
  const int64_t total = static_cast<int64_t>(p.n_layers) * p.batch * t.heads * vec_per_row;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int v = static_cast<int>(i % vec_per_row);
    const int64_t line = i / vec_per_row;  // (layer, slot, head)
    const int h = static_cast<int>(line % t.heads);
    const int64_t lb = line / t.heads;
    const int b = static_cast<int>(lb % p.batch);
    const int at = p.pos[p.pos_count == 1 ? 0 : b];
    if (at < 0 || at >= p.seq) continue;
    const char* src = static_cast<const char*>(t.src) + line * t.row_bytes;
    char* dst = static_cast<char*>(t.dst) + ((lb * t.heads + h) * p.seq + at) * t.row_bytes;
    switch (vec) {
      case 16: copy_vec<uint4>(dst, src, v); break;
      case 8: copy_vec<uint2>(dst, src, v); break;
      case 4: copy_vec<uint32_t>(dst, src, v); break;
      case 2: copy_vec<uint16_t>(dst, src, v); break;
      default: copy_vec<uint8_t>(dst, src, v); break;
    }
  }
}

// Widest power-of-two vector (<= 16 bytes) that divides the row and matches
// both base pointers.
int vector_bytes(const jpt_line_tensor& t) {
  for (int v = 16; v > 1; v >>= 1)
    if (t.row_bytes % v == 0 && aligned(t.dst, v) && aligned(t.src, v)) return v;
  return 1;
}

// ---- fused quantiser -------------------------------------------------------

struct QuantParams {
  jpt_quant_append_args a;
  // paged destination (jpt_paged_append_quant_i8): rows are addressed through
  // `indices` (3, stride) instead of pos; its first n_active columns count, or
  // its first *n_active_dev when that is set
  const int32_t* indices;
  const int32_t* n_active_dev;
  int32_t stride, total_pages, page_size;
};

template <bool ROUND_BF16>
__device__ __forceinline__ float rnd(float x) {
  return ROUND_BF16 ? round_to_bf16(x) : x;
}

// One pair of apply_rotary_emb: (a + bi)(c + si), one rounding per op and no
// fused multiply-add, then rounded to the tensor's dtype.
__device__ __forceinline__ void rotate_pair(float& a, float& b, float c, float s, bool to_bf16) {
#pragma clang fp contract(off)  // the products are rounded before they are combined
  const float ac = a * c, bs = b * s, as = a * s, bc = b * c;
  const float re = ac - bs;
  const float im = as + bc;
  a = to_bf16 ? round_to_bf16(re) : re;
  b = to_bf16 ? round_to_bf16(im) : im;
}

// One workgroup per (token, tensor): blockIdx.x = token (slot, or active
// index j when paged), blockIdx.y = 0 for K, 1 for V.  The op order is the
// reference's, each op rounded to the scale dtype:
//   trunc: a = absmax; s = a / 127;             q = x / s;      code = trunc(q)
//   rne:   a = max(absmax, eps); s = a / 127; r = 1 / s; q = x * r;
//          code = clamp(rint(q), -128, 127)
template <bool BF16_MATH>
__global__ void __launch_bounds__(256) quant_append_kernel(QuantParams p) {
  const jpt_quant_append_args& a = p.a;
  const bool paged = p.indices != nullptr;
  const int tok = blockIdx.x;
  if (paged && p.n_active_dev && tok >= *p.n_active_dev) return;  // whole workgroup
  const int b = paged ? p.indices[2 * p.stride + tok] : tok;
  if (b < 0 || b >= a.batch) return;
  const bool is_v = blockIdx.y == 1;
  const void* src = is_v ? a.new_v : a.new_k;
  int8_t* cache = static_cast<int8_t*>(is_v ? a.cache_v : a.cache_k);
  void* scale_out = is_v ? a.v_scale : a.k_scale;
  int8_t* stash = static_cast<int8_t*>(is_v ? a.out_v : a.out_k);
  void* stash_scale = is_v ? a.out_v_scale : a.out_k_scale;

  const int H = a.heads, D = a.dim, HD = H * D;
  const int groups = a.scale_heads;           // 1 or H
  const int per_group = HD / groups;          // elements sharing one scale
  const int64_t src_base = static_cast<int64_t>(b) * HD;

  __shared__ float s_red[4];
  __shared__ float s_scale[64 + 1];  // per group (heads <= 64 when per-head)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // element i of the token, rotated when this is the key side and factors are given
  const float* rope = is_v ? nullptr : a.rope;
  auto element = [&](int i) -> float {
    if (!rope) return load_as_f32(src, src_base + i, a.in_dtype);
    float x0 = load_as_f32(src, src_base + (i & ~1), a.in_dtype);
    float x1 = load_as_f32(src, src_base + (i | 1), a.in_dtype);
    const float2 cs = *reinterpret_cast<const float2*>(rope + (static_cast<int64_t>(b) * (D / 2) + (i % D) / 2) * 2);
    rotate_pair(x0, x1, cs.x, cs.y, a.in_dtype == JPT_BF16);
    return (i & 1) ? x1 : x0;
  };

  for (int g = 0; g < groups; ++g) {
    float m = 0.f;
    for (int i = threadIdx.x; i < per_group; i += blockDim.x)
      m = fmaxf(m, fabsf(element(g * per_group + i)));
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

  // destination of this token's rows
  int at, page = 0;
  bool write_cache = cache != nullptr;
  if (paged) {
    page = p.indices[tok];
    const int tok_index = p.indices[p.stride + tok];  // j * page_size + offset in the page
    at = tok_index % p.page_size;
    write_cache = write_cache && page >= 0 && page < p.total_pages && tok_index >= 0;
  } else {
    at = a.pos ? a.pos[a.pos_count == 1 ? 0 : b] : 0;
    write_cache = write_cache && at >= 0 && at < a.seq;
  }

  for (int i = threadIdx.x; i < HD; i += blockDim.x) {
    const int h = i / D, d = i - h * D;
    const float s = s_scale[groups == 1 ? 0 : h];
    const float x = element(i);
    int code;
    if (a.rounding == JPT_ROUND_TRUNC) {
      const float q = rnd<BF16_MATH>(x / s);
      code = (q != q) ? 0 : static_cast<int>(q);  // 0/0 -> 0; cast truncates
    } else {
      const float r = rnd<BF16_MATH>(1.0f / s);
      const float q = rnd<BF16_MATH>(x * r);
      code = static_cast<int>(fminf(fmaxf(rintf(q), -128.f), 127.f));
    }
    const int8_t c = static_cast<int8_t>(code);
    if (stash) stash[src_base + i] = c;
    if (write_cache) {
      const int64_t row = paged
          ? (static_cast<int64_t>(h) * p.total_pages + page) * p.page_size + at
          : (static_cast<int64_t>(b) * H + h) * a.seq + at;
      cache[row * D + d] = c;
    }
  }
  if (threadIdx.x < groups) {
    const int g = threadIdx.x;
    const float s = s_scale[g];
    if (stash_scale) store_from_f32(stash_scale, static_cast<int64_t>(b) * groups + g, a.scale_dtype, s);
    if (write_cache && scale_out) {
      const int64_t idx = paged
          ? (static_cast<int64_t>(g) * p.total_pages + page) * p.page_size + at
          : (static_cast<int64_t>(b) * groups + g) * a.seq + at;
      store_from_f32(scale_out, idx, a.scale_dtype, s);
    }
  }
}

// The same computation for the common shapes: bf16 input, heads * dim ==
// M * 1024; a thread keeps M runs of four elements in registers between the
// absmax pass and the quantise pass, and stores codes four at a time.
template <bool BF16_MATH, int M>
__global__ void __launch_bounds__(256) quant_append_vec_kernel(QuantParams p) {
  const jpt_quant_append_args& a = p.a;
  const bool paged = p.indices != nullptr;
  const int tok = blockIdx.x;
  if (paged && p.n_active_dev && tok >= *p.n_active_dev) return;  // whole workgroup
  const int b = paged ? p.indices[2 * p.stride + tok] : tok;
  if (b < 0 || b >= a.batch) return;
  const bool is_v = blockIdx.y == 1;
  const uint16_t* src = static_cast<const uint16_t*>(is_v ? a.new_v : a.new_k);
  int8_t* cache = static_cast<int8_t*>(is_v ? a.cache_v : a.cache_k);
  void* scale_out = is_v ? a.v_scale : a.k_scale;
  int8_t* stash = static_cast<int8_t*>(is_v ? a.out_v : a.out_k);
  void* stash_scale = is_v ? a.out_v_scale : a.out_k_scale;
  const int H = a.heads, D = a.dim, HD = H * D;
  const int groups = a.scale_heads;  // 1 or H
  const int64_t src_base = static_cast<int64_t>(b) * HD;

  // destination of this token's rows (read early: the loads overlap)
  int at, page = 0;
  bool write_cache = cache != nullptr;
  if (paged) {
    page = p.indices[tok];
    const int tok_index = p.indices[p.stride + tok];  // j * page_size + offset in the page
    at = tok_index % p.page_size;
    write_cache = write_cache && page >= 0 && page < p.total_pages && tok_index >= 0;
  } else {
    at = a.pos ? a.pos[a.pos_count == 1 ? 0 : b] : 0;
    write_cache = write_cache && at >= 0 && at < a.seq;
  }
  // run c of this thread: elements i0 .. i0 + 3, all of one head
  float x[M][4], m[M];
#pragma unroll
  for (int c = 0; c < M; ++c) {
    const int i0 = 4 * (threadIdx.x + 256 * c);
    const uint2 raw = *reinterpret_cast<const uint2*>(src + src_base + i0);
    x[c][0] = __uint_as_float(raw.x << 16);
    x[c][1] = __uint_as_float(raw.x & 0xffff0000u);
    x[c][2] = __uint_as_float(raw.y << 16);
    x[c][3] = __uint_as_float(raw.y & 0xffff0000u);
    if (!is_v && a.rope) {  // the run's two pairs: elements d, d + 1 and d + 2, d + 3 of the head
      const int d = i0 % D;
      const float4 cs = *reinterpret_cast<const float4*>(a.rope + (static_cast<int64_t>(b) * (D / 2) + d / 2) * 2);
      rotate_pair(x[c][0], x[c][1], cs.x, cs.y, true);
      rotate_pair(x[c][2], x[c][3], cs.z, cs.w, true);
    }
    m[c] = fmaxf(fmaxf(fabsf(x[c][0]), fabsf(x[c][1])), fmaxf(fabsf(x[c][2]), fabsf(x[c][3])));
  }

  __shared__ float s_red[4];
  float amax[M];
  if (groups == 1) {
    float all = m[0];
#pragma unroll
    for (int c = 1; c < M; ++c) all = fmaxf(all, m[c]);
    for (int off = 32; off > 0; off >>= 1) all = fmaxf(all, __shfl_xor(all, off));
    if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = all;
    __syncthreads();
    all = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
#pragma unroll
    for (int c = 0; c < M; ++c) amax[c] = all;
  } else {
    // a head's D / 4 threads of a run are consecutive; D / 4 is a power of two <= 64
#pragma unroll
    for (int c = 0; c < M; ++c) {
      for (int off = D / 8; off > 0; off >>= 1) m[c] = fmaxf(m[c], __shfl_xor(m[c], off));
      amax[c] = m[c];
    }
  }
#pragma unroll
  for (int c = 0; c < M; ++c) {
    const int i0 = 4 * (threadIdx.x + 256 * c);
    const int h = i0 / D, d = i0 - h * D;
    float am = amax[c];
    if (a.rounding == JPT_ROUND_RNE) am = fmaxf(am, rnd<BF16_MATH>(1e-5f));
    const float s = rnd<BF16_MATH>(am / 127.0f);
    int code[4];
    if (a.rounding == JPT_ROUND_TRUNC) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float q = rnd<BF16_MATH>(x[c][i] / s);
        code[i] = (q != q) ? 0 : static_cast<int>(q);  // 0/0 -> 0; cast truncates
      }
    } else {
      const float r = rnd<BF16_MATH>(1.0f / s);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float q = rnd<BF16_MATH>(x[c][i] * r);
        code[i] = static_cast<int>(fminf(fmaxf(rintf(q), -128.f), 127.f));
      }
    }
    const uint32_t packed = (static_cast<uint32_t>(code[0]) & 0xffu) | ((static_cast<uint32_t>(code[1]) & 0xffu) << 8) |
                            ((static_cast<uint32_t>(code[2]) & 0xffu) << 16) | (static_cast<uint32_t>(code[3]) << 24);
    if (stash) *reinterpret_cast<uint32_t*>(stash + src_base + i0) = packed;
    if (write_cache) {
      const int64_t row = paged
          ? (static_cast<int64_t>(h) * p.total_pages + page) * p.page_size + at
          : (static_cast<int64_t>(b) * H + h) * a.seq + at;
      *reinterpret_cast<uint32_t*>(cache + row * D + d) = packed;
    }
    // one thread per scale group writes the scale
    if (groups == 1 ? (c == 0 && threadIdx.x == 0) : d == 0) {
      const int g = groups == 1 ? 0 : h;
      if (stash_scale) store_from_f32(stash_scale, static_cast<int64_t>(b) * groups + g, a.scale_dtype, s);
      if (write_cache && scale_out) {
        const int64_t idx = paged
            ? (static_cast<int64_t>(g) * p.total_pages + page) * p.page_size + at
            : (static_cast<int64_t>(b) * groups + g) * a.seq + at;
        store_from_f32(scale_out, idx, a.scale_dtype, s);
      }
    }
  }
}

int32_t check_quant_common(int32_t heads, int32_t dim, int32_t in_dtype,
                           int32_t scale_dtype, int32_t scale_heads,
                           int32_t rounding) {
  JPT_REQUIRE(heads > 0 && dim > 0, "heads and dim must be positive");
  JPT_REQUIRE(in_dtype == JPT_BF16 || in_dtype == JPT_F32, "in_dtype must be bf16 or f32");
  JPT_REQUIRE(scale_dtype == in_dtype || scale_dtype == JPT_F32,
              "scale_dtype must equal in_dtype or be f32");
  JPT_REQUIRE(scale_heads == 1 || scale_heads == heads, "scale_heads must be 1 or heads");
  JPT_REQUIRE(scale_heads <= 64, "per-head scales support at most 64 heads");
  JPT_REQUIRE(rounding == JPT_ROUND_TRUNC || rounding == JPT_ROUND_RNE, "bad rounding mode");
  return JPT_OK;
}

// (rows, heads, dim) rotated by (rows, dim / 2, 2); a thread takes one pair
template <typename T>
__global__ void __launch_bounds__(256)
rope_kernel(T* out, const T* x, const float* freqs, int64_t pairs, int heads, int half) {
  const int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (i >= pairs) return;
  const int64_t row = i / (static_cast<int64_t>(heads) * half);
  const int p = static_cast<int>(i % half);
  const float2 cs = *reinterpret_cast<const float2*>(freqs + (row * half + p) * 2);
  constexpr bool kBf16 = sizeof(T) == 2;
  float a = kBf16 ? bf16_bits_to_f32(static_cast<uint16_t>(x[2 * i])) : static_cast<float>(x[2 * i]);
  float b = kBf16 ? bf16_bits_to_f32(static_cast<uint16_t>(x[2 * i + 1])) : static_cast<float>(x[2 * i + 1]);
  rotate_pair(a, b, cs.x, cs.y, false);
  out[2 * i] = kBf16 ? static_cast<T>(f32_to_bf16_bits(a)) : static_cast<T>(a);
  out[2 * i + 1] = kBf16 ? static_cast<T>(f32_to_bf16_bits(b)) : static_cast<T>(b);
}

int32_t launch_quant(const QuantParams& p, int32_t tokens, hipStream_t stream) {
  if (tokens == 0) return JPT_OK;
  dim3 grid(tokens, 2);
  const jpt_quant_append_args& a = p.a;
  const int d4 = a.dim / 4;
  const int runs = a.heads * a.dim / 1024;  // runs of four elements per thread
  const bool vec = a.in_dtype == JPT_BF16 && a.heads * a.dim % 1024 == 0 && (runs == 1 || runs == 2 || runs == 4) &&
                   a.dim % 4 == 0 &&
                   (a.scale_heads == 1 || (d4 <= 64 && (d4 & (d4 - 1)) == 0)) &&
                   aligned(a.new_k, 8) && aligned(a.new_v, 8) && aligned(a.out_k, 4) && aligned(a.out_v, 4) &&
                   aligned(a.cache_k, 4) && aligned(a.cache_v, 4) && aligned(a.rope, 16);
  if (vec) {
    const bool bf = a.scale_dtype == JPT_BF16;
#define JPT_LAUNCH_VEC(M)                                                                          \
  if (bf) hipLaunchKernelGGL((quant_append_vec_kernel<true, M>), grid, dim3(256), 0, stream, p);   \
  else hipLaunchKernelGGL((quant_append_vec_kernel<false, M>), grid, dim3(256), 0, stream, p)
    if (runs == 1) { JPT_LAUNCH_VEC(1); }
    else if (runs == 2) { JPT_LAUNCH_VEC(2); }
    else { JPT_LAUNCH_VEC(4); }
#undef JPT_LAUNCH_VEC
    return launch_status("quant_append_vec_kernel");
  }
  if (p.a.scale_dtype == JPT_BF16)
    hipLaunchKernelGGL(quant_append_kernel<true>, grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(quant_append_kernel<false>, grid, dim3(256), 0, stream, p);
  return launch_status("quant_append_kernel");
}

}  // namespace
}  // namespace jpt

extern "C" {

int32_t jpt_kv_scatter_lines(const jpt_line_tensor* tensors, int32_t n_tensors,
                             const int32_t* pos, int32_t pos_count,
                             int32_t n_layers, int32_t batch, int32_t seq,
                             void* stream) {
  using namespace jpt;
  JPT_REQUIRE(tensors != nullptr && pos != nullptr, "NULL argument");
  JPT_REQUIRE(n_tensors >= 1 && n_tensors <= JPT_MAX_LINE_TENSORS, "n_tensors must be 1..%d", JPT_MAX_LINE_TENSORS);
  JPT_REQUIRE(n_layers > 0 && batch > 0 && seq > 0, "n_layers, batch, seq must be positive");
  JPT_REQUIRE(pos_count == 1 || pos_count == batch, "pos_count must be 1 or batch");
  LineParams p{};
  int64_t most = 0;
  for (int i = 0; i < n_tensors; ++i) {
    JPT_REQUIRE(tensors[i].dst && tensors[i].src, "tensor %d has a NULL pointer", i);
    JPT_REQUIRE(tensors[i].heads > 0 && tensors[i].row_bytes > 0, "tensor %d: heads and row_bytes must be positive", i);
    p.t[i] = tensors[i];
    p.vec[i] = vector_bytes(tensors[i]);
    const int64_t n = static_cast<int64_t>(n_layers) * batch * tensors[i].heads * (tensors[i].row_bytes / p.vec[i]);
    most = n > most ? n : most;
  }
  p.pos = pos;
  p.pos_count = pos_count;
  p.n_layers = n_layers;
  p.batch = batch;
  p.seq = seq;
  int64_t blocks = (most + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  dim3 grid(static_cast<unsigned>(blocks), n_tensors);
  hipLaunchKernelGGL(scatter_lines_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), p);
  return launch_status("scatter_lines_kernel");
}

int32_t jpt_kv_append_quant_i8(const jpt_quant_append_args* args, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(args != nullptr, "args is NULL");
  const jpt_quant_append_args& a = *args;
  JPT_REQUIRE(a.new_k && a.new_v, "new_k/new_v are NULL");
  JPT_REQUIRE(a.batch > 0, "batch must be positive");
  int32_t st = check_quant_common(a.heads, a.dim, a.in_dtype, a.scale_dtype, a.scale_heads, a.rounding);
  if (st != JPT_OK) return st;
  JPT_REQUIRE(!a.rope || (a.dim % 2 == 0 && aligned(a.rope, 8)), "rope needs an even dim and 8-byte aligned factors");
  const bool to_cache = a.cache_k != nullptr || a.cache_v != nullptr;
  if (to_cache) {
    JPT_REQUIRE(a.cache_k && a.cache_v && a.k_scale && a.v_scale, "cache_k, cache_v, k_scale, v_scale must all be set");
    JPT_REQUIRE(a.pos != nullptr && (a.pos_count == 1 || a.pos_count == a.batch), "pos must hold 1 or batch entries");
    JPT_REQUIRE(a.seq > 0, "seq must be positive");
  } else {
    JPT_REQUIRE(a.out_k && a.out_v && a.out_k_scale && a.out_v_scale, "nothing to write: cache_* and out_* are NULL");
  }
  QuantParams p{};
  p.a = a;
  return launch_quant(p, a.batch, static_cast<hipStream_t>(stream));
}

int32_t jpt_rope(void* out, const void* x, const float* freqs, int32_t rows, int32_t heads, int32_t dim,
                 int32_t dtype, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(out && x && freqs, "NULL argument");
  JPT_REQUIRE(rows >= 0 && heads > 0 && dim > 0 && dim % 2 == 0, "rows >= 0, heads > 0 and an even dim are needed");
  JPT_REQUIRE(dtype == JPT_BF16 || dtype == JPT_F32, "dtype must be bf16 or f32");
  JPT_REQUIRE(aligned(freqs, 8), "freqs must be 8-byte aligned");
  const int64_t pairs = static_cast<int64_t>(rows) * heads * (dim / 2);
  if (pairs == 0) return JPT_OK;
  const dim3 grid(static_cast<unsigned>((pairs + 255) / 256));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == JPT_BF16)
    hipLaunchKernelGGL(rope_kernel<uint16_t>, grid, dim3(256), 0, s, static_cast<uint16_t*>(out),
                       static_cast<const uint16_t*>(x), freqs, pairs, heads, dim / 2);
  else
    hipLaunchKernelGGL(rope_kernel<float>, grid, dim3(256), 0, s, static_cast<float*>(out),
                       static_cast<const float*>(x), freqs, pairs, heads, dim / 2);
  return launch_status("rope_kernel");
}

int32_t jpt_paged_append_quant_i8(const jpt_paged_quant_append_args* args, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(args != nullptr, "args is NULL");
  const jpt_paged_quant_append_args& g = *args;
  JPT_REQUIRE(g.new_k && g.new_v && g.pages_k && g.pages_v && g.k_scale_pages && g.v_scale_pages, "NULL tensor argument");
  const bool dev_count = g.n_active_dev != nullptr;
  if (dev_count) {
    JPT_REQUIRE(g.indices != nullptr && g.indices_stride >= 1 && g.indices_stride <= g.batch,
                "with n_active_dev, indices must be (3, indices_stride), indices_stride in 1..batch");
  } else {
    JPT_REQUIRE(g.n_active >= 0 && g.n_active <= g.batch, "n_active must be 0..batch");
    JPT_REQUIRE(g.n_active == 0 || g.indices != nullptr, "indices is NULL");
  }
  JPT_REQUIRE(g.total_pages > 0 && g.page_size > 0, "total_pages and page_size must be positive");
  JPT_REQUIRE(!g.rope || (g.dim % 2 == 0 && aligned(g.rope, 8)), "rope needs an even dim and 8-byte aligned factors");
  int32_t st = check_quant_common(g.heads, g.dim, g.in_dtype, g.scale_dtype, g.scale_heads, g.rounding);
  if (st != JPT_OK) return st;
  QuantParams p{};
  p.a.new_k = g.new_k;
  p.a.new_v = g.new_v;
  p.a.cache_k = g.pages_k;
  p.a.cache_v = g.pages_v;
  p.a.k_scale = g.k_scale_pages;
  p.a.v_scale = g.v_scale_pages;
  p.a.batch = g.batch;
  p.a.heads = g.heads;
  p.a.dim = g.dim;
  p.a.in_dtype = g.in_dtype;
  p.a.scale_dtype = g.scale_dtype;
  p.a.scale_heads = g.scale_heads;
  p.a.rounding = g.rounding;
  p.a.rope = g.rope;
  p.indices = g.indices;
  p.n_active_dev = g.n_active_dev;
  p.stride = dev_count ? g.indices_stride : g.n_active;
  p.total_pages = g.total_pages;
  p.page_size = g.page_size;
  return launch_quant(p, dev_count ? g.indices_stride : g.n_active, static_cast<hipStream_t>(stream));
}

}  // extern "C"
