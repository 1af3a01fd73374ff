// Paged KV cache data movement: prefill insert, per-step row append and the
// page-table gather.  Pages are (heads, total_pages, page_size, row_bytes).
// All three are HBM-bound copies; a thread moves one 16-byte (or narrower)
// vector, consecutive threads move consecutive bytes of a row.
#include "common.h"

namespace jpt {
namespace {

template <typename V>
__device__ __forceinline__ V zero_of();
template <> __device__ __forceinline__ uint4 zero_of<uint4>() { return make_uint4(0, 0, 0, 0); }
template <> __device__ __forceinline__ uint2 zero_of<uint2>() { return make_uint2(0, 0); }
template <> __device__ __forceinline__ uint32_t zero_of<uint32_t>() { return 0u; }
template <> __device__ __forceinline__ uint16_t zero_of<uint16_t>() { return 0; }
template <> __device__ __forceinline__ uint8_t zero_of<uint8_t>() { return 0; }

int pick_vec(int row_bytes, std::initializer_list<const void*> ptrs) {
  for (int v = 16; v > 1; v >>= 1) {
    bool ok = row_bytes % v == 0;
    for (const void* p : ptrs) ok = ok && aligned(p, v);
    if (ok) return v;
  }
  return 1;
}

#define JPT_DISPATCH_VEC(vec, KERNEL, grid, stream, ...)                                   \
  switch (vec) {                                                                            \
    case 16: hipLaunchKernelGGL(KERNEL<uint4>, grid, dim3(256), 0, stream, __VA_ARGS__); break;    \
    case 8: hipLaunchKernelGGL(KERNEL<uint2>, grid, dim3(256), 0, stream, __VA_ARGS__); break;     \
    case 4: hipLaunchKernelGGL(KERNEL<uint32_t>, grid, dim3(256), 0, stream, __VA_ARGS__); break;  \
    case 2: hipLaunchKernelGGL(KERNEL<uint16_t>, grid, dim3(256), 0, stream, __VA_ARGS__); break;  \
    default: hipLaunchKernelGGL(KERNEL<uint8_t>, grid, dim3(256), 0, stream, __VA_ARGS__); break;  \
  }

// pages[h, page_ids[p], t, :] = (p*ps + t < seq_len) ? src[h, p*ps + t, :] : 0
// grid.y = 0 for K, 1 for V.
template <typename V>
__global__ void __launch_bounds__(256)
paged_insert_kernel(void* pages_k, void* pages_v, const void* src_k, const void* src_v,
                    const int32_t* page_ids, int n_pages, int seq_len, int heads,
                    int total_pages, int page_size, int row_bytes) {
  V* pages = static_cast<V*>(blockIdx.y ? pages_v : pages_k);
  const V* src = static_cast<const V*>(blockIdx.y ? src_v : src_k);
  const int vpr = row_bytes / sizeof(V);
  const int64_t total = static_cast<int64_t>(heads) * n_pages * page_size * vpr;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int v = static_cast<int>(i % vpr);
    int64_t r = i / vpr;
    const int t = static_cast<int>(r % page_size);
    r /= page_size;
    const int pg = static_cast<int>(r % n_pages);
    const int h = static_cast<int>(r / n_pages);
    const int page = page_ids[pg];
    if (page < 0 || page >= total_pages) continue;
    const int tok = pg * page_size + t;
    const V val = tok < seq_len ? src[(static_cast<int64_t>(h) * seq_len + tok) * vpr + v]
                                : zero_of<V>();
    pages[((static_cast<int64_t>(h) * total_pages + page) * page_size + t) * vpr + v] = val;
  }
}

// pages[h, page_j, tok_j % ps, :] = src[slot_j, h, 0, :].  `indices` is
// (3, stride); the column count is n_active, or *n_active_dev when that is set.
template <typename V>
__global__ void __launch_bounds__(256)
paged_append_kernel(void* pages_k, void* pages_v, const void* src_k, const void* src_v,
                    const int32_t* indices, int stride, int n_active, const int32_t* n_active_dev,
                    int batch, int heads, int total_pages, int page_size, int row_bytes) {
  V* pages = static_cast<V*>(blockIdx.y ? pages_v : pages_k);
  const V* src = static_cast<const V*>(blockIdx.y ? src_v : src_k);
  const int vpr = row_bytes / sizeof(V);
  if (n_active_dev) n_active = min(max(*n_active_dev, 0), stride);
  const int64_t total = static_cast<int64_t>(n_active) * heads * vpr;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int v = static_cast<int>(i % vpr);
    const int64_t r = i / vpr;
    const int h = static_cast<int>(r % heads);
    const int j = static_cast<int>(r / heads);
    const int page = indices[j];
    const int t = indices[stride + j] % page_size;
    const int slot = indices[2 * stride + j];
    if (page < 0 || page >= total_pages || slot < 0 || slot >= batch || t < 0) continue;
    pages[((static_cast<int64_t>(h) * total_pages + page) * page_size + t) * vpr + v] =
        src[(static_cast<int64_t>(slot) * heads + h) * vpr + v];
  }
}

// dst[h, t, :] = pages[h, page_row[t / ps], t % ps, :], t < length
template <typename V>
__global__ void __launch_bounds__(256)
paged_gather_kernel(void* dst_, const void* pages_, const int32_t* page_row, int length,
                    int heads, int total_pages, int page_size, int row_bytes) {
  V* dst = static_cast<V*>(dst_);
  const V* pages = static_cast<const V*>(pages_);
  const int vpr = row_bytes / sizeof(V);
  const int64_t total = static_cast<int64_t>(heads) * length * vpr;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int v = static_cast<int>(i % vpr);
    const int64_t r = i / vpr;
    const int t = static_cast<int>(r % length);
    const int h = static_cast<int>(r / length);
    const int page = page_row[t / page_size];
    if (page < 0 || page >= total_pages) continue;
    dst[i] = pages[((static_cast<int64_t>(h) * total_pages + page) * page_size + t % page_size) * vpr + v];
  }
}

unsigned blocks_for(int64_t threads) {
  int64_t b = (threads + 255) / 256;
  return static_cast<unsigned>(b < 1 ? 1 : (b > 65535 ? 65535 : b));
}

}  // namespace
}  // namespace jpt

extern "C" {

int32_t jpt_paged_insert(void* pages_k, void* pages_v, const void* src_k,
                         const void* src_v, const int32_t* page_ids,
                         int32_t n_pages, int32_t seq_len, int32_t heads,
                         int32_t total_pages, int32_t page_size,
                         int32_t row_bytes, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(pages_k && pages_v && src_k && src_v, "NULL tensor argument");
  JPT_REQUIRE(heads > 0 && total_pages > 0 && page_size > 0 && row_bytes > 0, "heads, total_pages, page_size, row_bytes must be positive");
  JPT_REQUIRE(n_pages >= 0 && seq_len >= 0, "negative n_pages or seq_len");
  JPT_REQUIRE(static_cast<int64_t>(n_pages) * page_size >= seq_len, "%d pages of %d tokens cannot hold %d tokens", n_pages, page_size, seq_len);
  if (n_pages == 0) return JPT_OK;
  JPT_REQUIRE(page_ids != nullptr, "page_ids is NULL");
  const int vec = pick_vec(row_bytes, {pages_k, pages_v, src_k, src_v});
  dim3 grid(blocks_for(static_cast<int64_t>(heads) * n_pages * page_size * (row_bytes / vec)), 2);
  hipStream_t s = static_cast<hipStream_t>(stream);
  JPT_DISPATCH_VEC(vec, paged_insert_kernel, grid, s, pages_k, pages_v, src_k, src_v, page_ids,
                   n_pages, seq_len, heads, total_pages, page_size, row_bytes);
  return launch_status("paged_insert_kernel");
}

int32_t jpt_paged_append(void* pages_k, void* pages_v, const void* src_k,
                         const void* src_v, const int32_t* indices,
                         int32_t n_active, int32_t batch, int32_t heads,
                         int32_t total_pages, int32_t page_size,
                         int32_t row_bytes, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(pages_k && pages_v && src_k && src_v, "NULL tensor argument");
  JPT_REQUIRE(batch > 0 && heads > 0 && total_pages > 0 && page_size > 0 && row_bytes > 0, "batch, heads, total_pages, page_size, row_bytes must be positive");
  JPT_REQUIRE(n_active >= 0 && n_active <= batch, "n_active must be 0..batch");
  if (n_active == 0) return JPT_OK;
  JPT_REQUIRE(indices != nullptr, "indices is NULL");
  const int vec = pick_vec(row_bytes, {pages_k, pages_v, src_k, src_v});
  dim3 grid(blocks_for(static_cast<int64_t>(n_active) * heads * (row_bytes / vec)), 2);
  hipStream_t s = static_cast<hipStream_t>(stream);
  JPT_DISPATCH_VEC(vec, paged_append_kernel, grid, s, pages_k, pages_v, src_k, src_v, indices,
                   n_active, n_active, static_cast<const int32_t*>(nullptr), batch, heads, total_pages,
                   page_size, row_bytes);
  return launch_status("paged_append_kernel");
}

int32_t jpt_paged_append_dev(void* pages_k, void* pages_v, const void* src_k,
                             const void* src_v, const int32_t* indices,
                             int32_t indices_stride, const int32_t* n_active_dev,
                             int32_t batch, int32_t heads, int32_t total_pages,
                             int32_t page_size, int32_t row_bytes, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(pages_k && pages_v && src_k && src_v && indices && n_active_dev, "NULL argument");
  JPT_REQUIRE(batch > 0 && heads > 0 && total_pages > 0 && page_size > 0 && row_bytes > 0, "batch, heads, total_pages, page_size, row_bytes must be positive");
  JPT_REQUIRE(indices_stride >= 1, "indices_stride must be positive");
  const int vec = pick_vec(row_bytes, {pages_k, pages_v, src_k, src_v});
  // sized for every column; blocks past the device-side count find nothing to do
  dim3 grid(blocks_for(static_cast<int64_t>(indices_stride) * heads * (row_bytes / vec)), 2);
  hipStream_t s = static_cast<hipStream_t>(stream);
  JPT_DISPATCH_VEC(vec, paged_append_kernel, grid, s, pages_k, pages_v, src_k, src_v, indices,
                   indices_stride, 0, n_active_dev, batch, heads, total_pages, page_size, row_bytes);
  return launch_status("paged_append_kernel");
}

int32_t jpt_paged_gather(void* dst, const void* pages, const int32_t* page_row,
                         int32_t max_pages, int32_t length, int32_t heads,
                         int32_t total_pages, int32_t page_size,
                         int32_t row_bytes, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(dst && pages && page_row, "NULL argument");
  JPT_REQUIRE(heads > 0 && total_pages > 0 && page_size > 0 && row_bytes > 0, "heads, total_pages, page_size, row_bytes must be positive");
  JPT_REQUIRE(length >= 0, "negative length");
  JPT_REQUIRE(max_pages > 0 && static_cast<int64_t>(length) <= static_cast<int64_t>(max_pages) * page_size,
              "length %d is past the %d pages of the row", length, max_pages);
  if (length == 0) return JPT_OK;
  const int vec = pick_vec(row_bytes, {dst, pages});
  dim3 grid(blocks_for(static_cast<int64_t>(heads) * length * (row_bytes / vec)));
  hipStream_t s = static_cast<hipStream_t>(stream);
  JPT_DISPATCH_VEC(vec, paged_gather_kernel, grid, s, dst, pages, page_row, length, heads,
                   total_pages, page_size, row_bytes);
  return launch_status("paged_gather_kernel");
}

}  // extern "C"
