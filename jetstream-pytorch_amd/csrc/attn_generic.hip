// Shape-generic decode attention: any head_dim <= 512, any number of query
// rows, bf16/f32/int8 keys, optional scales, additive mask, page table and
// fused new-token term.  One wavefront per (slot, q head, q row); scores of a
// tile of positions go through LDS, the online softmax is carried in
// registers.  It is the path for shapes the MFMA kernel does not take (tiny
// test shapes, prefill-shaped calls, f32 caches) and is not tuned; it also
// serves as a second implementation to cross-check the MFMA kernel on the GPU.
#include <math.h>

#include "attn_common.h"

namespace jpt {
namespace {

constexpr int kTile = 1024;
constexpr int kMaxDimPerLane = 8;  // head_dim <= 512

__device__ __forceinline__ float wave_max(float v) {
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

__global__ void __launch_bounds__(64) attn_generic_kernel(jpt_attn_args a, int mode) {
  __shared__ float sc[kTile];
  __shared__ float qs[64 * kMaxDimPerLane];

  const int lane = threadIdx.x;
  const int D = a.dim, T = a.q_rows;
  const int row = blockIdx.x;
  const int t = row % T;
  const int hq = (row / T) % a.q_heads;
  const int b = row / (T * a.q_heads);
  const int rep = a.q_heads / a.kv_heads;
  const int hkv = hq / rep;
  const int hs = a.scale_heads == 1 ? 0 : hkv;
  const bool paged = mode == kPaged;
  const int ps = paged ? a.page_size : 1;

  int n = a.lengths ? a.lengths[b] : a.seq;
  const int cap = paged ? a.max_pages * a.page_size : a.seq;
  n = n < 0 ? 0 : (n > cap ? cap : n);

  for (int d = lane; d < D; d += 64)
    qs[d] = load_as_f32(a.q, static_cast<int64_t>(row) * D + d, a.q_dtype);
  __syncthreads();

  float acc[kMaxDimPerLane];
#pragma unroll
  for (int i = 0; i < kMaxDimPerLane; ++i) acc[i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // Row (in units of head rows) of position `tok` in the key/value tensor and
  // in the scale tensor.
  auto kv_row = [&](int tok, int64_t* srow) -> int64_t {
    if (paged) {
      int page = a.page_table[static_cast<int64_t>(b) * a.max_pages + tok / ps];
      page = min(max(page, 0), a.total_pages - 1);  // whatever the table holds, stay inside the pool
      const int64_t in_page = static_cast<int64_t>(page) * ps + tok % ps;
      *srow = static_cast<int64_t>(hs) * a.total_pages * ps + in_page;
      return static_cast<int64_t>(hkv) * a.total_pages * ps + in_page;
    }
    *srow = (static_cast<int64_t>(b) * a.scale_heads + hs) * a.seq + tok;
    return (static_cast<int64_t>(b) * a.kv_heads + hkv) * a.seq + tok;
  };

  for (int ts = 0; ts < n; ts += kTile) {
    const int nt = min(kTile, n - ts);
    float tmax = -INFINITY;
    for (int tt = lane; tt < nt; tt += 64) {
      int64_t srow;
      const int64_t krow = kv_row(ts + tt, &srow);
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot += qs[d] * load_as_f32(a.k, krow * D + d, a.kv_dtype);
      float s = dot * a.sm_scale;
      if (a.k_scale) s *= load_as_f32(a.k_scale, srow, a.scale_dtype);
      if (a.mask)
        s += load_as_f32(a.mask, b * a.mask_stride_b + hq * a.mask_stride_h +
                                     t * a.mask_stride_t + ts + tt, a.mask_dtype);
      sc[tt] = s;
      tmax = fmaxf(tmax, s);
    }
    tmax = wave_max(tmax);
    const float m_new = fmaxf(m_run, tmax);
    if (m_new == -INFINITY) continue;  // everything so far is masked out
    const float alpha = expf(m_run - m_new);
    float lsum = 0.f;
    for (int tt = lane; tt < nt; tt += 64) {
      int64_t srow;
      kv_row(ts + tt, &srow);
      const float p = expf(sc[tt] - m_new);
      lsum += p;
      sc[tt] = a.v_scale ? p * load_as_f32(a.v_scale, srow, a.scale_dtype) : p;
    }
    l_run = l_run * alpha + wave_sum(lsum);
    m_run = m_new;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kMaxDimPerLane; ++i) acc[i] *= alpha;
    for (int tt = 0; tt < nt; ++tt) {
      int64_t srow;
      const int64_t vrow = kv_row(ts + tt, &srow);
      const float p = sc[tt];
#pragma unroll
      for (int i = 0; i < kMaxDimPerLane; ++i) {
        const int d = lane + 64 * i;
        if (d < D) acc[i] += p * load_as_f32(a.v, vrow * D + d, a.kv_dtype);
      }
    }
    __syncthreads();
  }

  if (a.new_k) {  // the step's own token, one more position
    const int64_t nrow = static_cast<int64_t>(b) * a.kv_heads + hkv;
    float part = 0.f;
    for (int d = lane; d < D; d += 64) part += qs[d] * load_as_f32(a.new_k, nrow * D + d, a.kv_dtype);
    float s = wave_sum(part) * a.sm_scale;
    float vs = 1.f;
    if (a.new_k_scale) {
      const int64_t si = static_cast<int64_t>(b) * a.scale_heads + hs;
      s *= load_as_f32(a.new_k_scale, si, a.scale_dtype);
      vs = load_as_f32(a.new_v_scale, si, a.scale_dtype);
    }
    const float m_new = fmaxf(m_run, s);
    const float alpha = expf(m_run - m_new);
    const float p = expf(s - m_new);
    l_run = l_run * alpha + p;
    m_run = m_new;
#pragma unroll
    for (int i = 0; i < kMaxDimPerLane; ++i) {
      const int d = lane + 64 * i;
      if (d < D) acc[i] = acc[i] * alpha + p * vs * load_as_f32(a.new_v, nrow * D + d, a.kv_dtype);
    }
  }

  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
#pragma unroll
  for (int i = 0; i < kMaxDimPerLane; ++i) {
    const int d = lane + 64 * i;
    if (d < D) store_from_f32(a.out, static_cast<int64_t>(row) * D + d, a.q_dtype, acc[i] * inv);
  }
  if (lane == 0) {
    if (a.out_max) a.out_max[row] = m_run;
    if (a.out_denom) a.out_denom[row] = l_run;
  }
}

__global__ void __launch_bounds__(256)
lse_merge_kernel(void* out, const void* o1, const float* m1, const float* l1,
                 const void* o2, const float* m2, const float* l2, int64_t rows,
                 int dim, int dtype) {
  const int64_t total = rows * dim;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = i / dim;
    const float g = fmaxf(m1[r], m2[r]);
    // a side that attended nothing has max = -inf; exp(-inf - g) = 0 unless
    // g is -inf too, in which case both weights are defined as 0
    const float alpha = g == -INFINITY ? 0.f : expf(m1[r] - g);
    const float beta = g == -INFINITY ? 0.f : expf(m2[r] - g);
    const float den = alpha * l1[r] + beta * l2[r];
    const float num = l1[r] * alpha * load_as_f32(o1, i, dtype) +
                      beta * load_as_f32(o2, i, dtype) * l2[r];
    store_from_f32(out, i, dtype, den > 0.f ? num / den : 0.f);
  }
}

}  // namespace

int32_t attn_generic_launch(const jpt_attn_args& a, AttnMode mode, hipStream_t stream) {
  JPT_REQUIRE(a.dim <= 64 * kMaxDimPerLane, "generic attention kernel supports head_dim <= %d", 64 * kMaxDimPerLane);
  const int64_t rows = static_cast<int64_t>(a.batch) * a.q_heads * a.q_rows;
  JPT_REQUIRE(rows < (1ll << 31), "too many query rows");
  hipLaunchKernelGGL(attn_generic_kernel, dim3(static_cast<unsigned>(rows)), dim3(64), 0, stream, a,
                     static_cast<int>(mode));
  return launch_status("attn_generic_kernel");
}

int32_t check_attn_args(const jpt_attn_args& a, AttnMode mode) {
  JPT_REQUIRE(a.q && a.k && a.v && a.out, "q, k, v, out must be set");
  JPT_REQUIRE(a.batch > 0 && a.q_heads > 0 && a.kv_heads > 0 && a.q_rows > 0 && a.dim > 0, "batch, heads, q_rows, dim must be positive");
  JPT_REQUIRE(a.q_heads % a.kv_heads == 0, "q_heads %d is not a multiple of kv_heads %d", a.q_heads, a.kv_heads);
  JPT_REQUIRE(a.q_dtype == JPT_BF16 || a.q_dtype == JPT_F32, "q_dtype must be bf16 or f32");
  JPT_REQUIRE(a.kv_dtype == JPT_BF16 || a.kv_dtype == JPT_F32 || a.kv_dtype == JPT_I8, "bad kv_dtype");
  JPT_REQUIRE((a.k_scale == nullptr) == (a.v_scale == nullptr), "k_scale and v_scale go together");
  if (a.k_scale) {
    JPT_REQUIRE(a.scale_dtype == JPT_BF16 || a.scale_dtype == JPT_F32, "scale_dtype must be bf16 or f32");
    JPT_REQUIRE(a.scale_heads == 1 || a.scale_heads == a.kv_heads, "scale_heads must be 1 or kv_heads");
  }
  JPT_REQUIRE((a.new_k == nullptr) == (a.new_v == nullptr), "new_k and new_v go together");
  if (a.new_k) {
    JPT_REQUIRE((a.new_k_scale != nullptr) == (a.k_scale != nullptr) && (a.new_v_scale != nullptr) == (a.k_scale != nullptr),
                "the new token carries scales exactly when the cache does");
    JPT_REQUIRE(a.q_rows == 1, "the fused new-token term needs q_rows == 1");
  }
  JPT_REQUIRE((a.new_k_raw == nullptr) == (a.new_v_raw == nullptr), "new_k_raw and new_v_raw go together");
  if (a.new_k_raw) {
    JPT_REQUIRE(a.kv_dtype == JPT_I8 && a.k_scale != nullptr, "new_k_raw is for an int8 cache with scales");
    JPT_REQUIRE(a.new_k && a.new_k_scale && a.new_v_scale, "new_k_raw needs new_k/new_v/new_k_scale/new_v_scale to write to");
    JPT_REQUIRE(a.new_rounding == JPT_ROUND_TRUNC || a.new_rounding == JPT_ROUND_RNE, "bad new_rounding");
  }
  JPT_REQUIRE(a.new_k_rope == nullptr || (a.new_k_raw != nullptr && a.dim % 2 == 0 && aligned(a.new_k_rope, 16)),
              "new_k_rope needs new_k_raw, an even dim and 16-byte aligned factors");
  if (a.mask) JPT_REQUIRE(a.mask_dtype == JPT_BF16 || a.mask_dtype == JPT_F32, "mask_dtype must be bf16 or f32");
  if (mode == kPaged) {
    JPT_REQUIRE(a.page_table && a.lengths, "paged attention needs page_table and lengths");
    JPT_REQUIRE(a.total_pages > 0 && a.page_size > 0 && a.max_pages > 0, "total_pages, page_size, max_pages must be positive");
    JPT_REQUIRE(a.mask == nullptr, "paged attention takes no mask");
    JPT_REQUIRE(!a.new_to_pages || a.new_k != nullptr, "new_to_pages needs the new token (new_k/new_v)");
  } else {
    JPT_REQUIRE(!a.new_to_pages, "new_to_pages is for the paged entry point");
    JPT_REQUIRE(a.seq > 0, "seq must be positive");
    JPT_REQUIRE(a.page_table == nullptr, "page_table given to a non-paged entry point");
    if (mode == kRagged) JPT_REQUIRE(a.lengths != nullptr, "ragged attention needs lengths");
  }
  return JPT_OK;
}

}  // namespace jpt

extern "C" {

int32_t jpt_lse_merge(void* out, const void* o1, const float* m1, const float* l1,
                      const void* o2, const float* m2, const float* l2, int64_t rows,
                      int32_t dim, int32_t dtype, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(out && o1 && m1 && l1 && o2 && m2 && l2, "NULL argument");
  JPT_REQUIRE(rows >= 0 && dim > 0, "rows must be >= 0 and dim positive");
  JPT_REQUIRE(dtype == JPT_BF16 || dtype == JPT_F32, "dtype must be bf16 or f32");
  if (rows == 0) return JPT_OK;
  int64_t blocks = (rows * dim + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(lse_merge_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), out, o1, m1, l1, o2, m2, l2, rows, dim, dtype);
  return launch_status("lse_merge_kernel");
}

}  // extern "C"
