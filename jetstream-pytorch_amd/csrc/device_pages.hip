// Device-resident page allocator and decode-state bookkeeping.
//
// PageAttentionManager (jetstream_pt/page_attention_manager.py:21-64, :145-177,
// :214-222) with the free list, the page table and the lengths in HBM.  Every
// method is one workgroup of 256 threads: the work is a few hundred integers,
// and one workgroup keeps the FIFO order of the reference (slots served in
// ascending order, requests in the order given) without any atomics - a
// slot's place in the hand-out order is a prefix sum over the slots before it.
// Kernels cannot raise; a request that cannot be served is skipped and leaves
// a bit in state[2]; a decode step whose page request fails drops that slot's
// token (page -1 in its column of update_indices and in its table cell)
// instead of writing it anywhere.  No index read from memory is used before it is checked
// against the array it addresses.
#include <algorithm>

#include "common.h"

namespace jpt {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ void raise(const jpt_dpam& d, int bit) { atomicOr(&d.state[2], bit); }

// Exclusive prefix sum of `x` over the workgroup's threads; *total gets the sum.
__device__ __forceinline__ int block_exclusive_scan(int x, int* total) {
  __shared__ int s_wave[kThreads / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = x;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int y = __shfl_up(incl, off);
    if (lane >= off) incl += y;
  }
  __syncthreads();  // s_wave may still be read from the previous call
  if (lane == 63) s_wave[wave] = incl;
  __syncthreads();
  int before = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < kThreads / 64; ++w) {
    if (w < wave) before += s_wave[w];
    sum += s_wave[w];
  }
  *total = sum;
  return before + incl - x;
}

__global__ void __launch_bounds__(kThreads)
dpam_init_kernel(jpt_dpam d, const int32_t* free_order) {
  const int64_t tid = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = tid; i < d.total_pages; i += step) d.ring[i] = free_order ? free_order[i] : static_cast<int32_t>(i);
  const int64_t cells = static_cast<int64_t>(d.batch) * d.max_pages;
  // the sentinel is the last page id, itself allocatable (:30-35)
  for (int64_t i = tid; i < cells; i += step) d.page_indices[i] = d.total_pages - 1;
  for (int64_t i = tid; i < d.batch; i += step) {
    d.lengths[i] = 0;
    d.n_alloc[i] = 0;
  }
  for (int64_t i = tid; i < 3 * static_cast<int64_t>(d.batch); i += step) d.update_indices[i] = 0;
  if (tid == 0) {
    d.state[0] = 0;
    d.state[1] = d.total_pages;
    d.state[2] = 0;
    d.state[3] = 0;
  }
}

// reserve_pages_insert (:42-52), requests served one after another.  The free
// list's head and count travel in registers (every thread computes the same
// values) and the requests are read kThreads at a time, so a request costs one
// memory round trip - ring to table row - and no barrier: rows and ring cells
// of different requests are disjoint, and a slot named twice is written twice
// by the same threads in request order.
__global__ void __launch_bounds__(kThreads)
dpam_reserve_insert_kernel(jpt_dpam d, const int32_t* slots, const int32_t* seq_lens, int n_req,
                           int slot_imm, int len_imm) {
  __shared__ int s_slot[kThreads], s_len[kThreads];
  int head = d.state[0], count = d.state[1];
  for (int r0 = 0; r0 < n_req; r0 += kThreads) {
    __syncthreads();  // the previous batch of requests has been read
    if (r0 + threadIdx.x < n_req) {
      s_slot[threadIdx.x] = slots ? slots[r0 + threadIdx.x] : slot_imm;
      s_len[threadIdx.x] = seq_lens ? seq_lens[r0 + threadIdx.x] : len_imm;
    }
    __syncthreads();
    const int n_here = min(kThreads, n_req - r0);
    for (int j = 0; j < n_here; ++j) {
      const int slot = s_slot[j], len = s_len[j];
      if (slot < 0 || slot >= d.batch || len < 0) {
        if (threadIdx.x == 0) raise(d, JPT_DPAM_BADARG);
        continue;
      }
      const int n = (len + d.page_size - 1) / d.page_size;
      if (n > d.max_pages) {
        if (threadIdx.x == 0) raise(d, JPT_DPAM_OVERFLOW);
        continue;
      }
      if (n > count) {
        if (threadIdx.x == 0) raise(d, JPT_DPAM_NOPAGES);
        continue;
      }
      int32_t* row = d.page_indices + static_cast<int64_t>(slot) * d.max_pages;
      for (int i = threadIdx.x; i < n; i += kThreads) row[i] = d.ring[(head + i) % d.total_pages];
      if (threadIdx.x == 0) {
        d.lengths[slot] = len;
        d.n_alloc[slot] = n;
      }
      head = (head + n) % d.total_pages;
      count -= n;
    }
  }
  if (threadIdx.x == 0) {
    d.state[0] = head;
    d.state[1] = count;
  }
}

// free_pages_resource (:214-222): the slot's pages go to the tail of the free
// list in row order; row back to the sentinel, length to 0.  Requests are read
// kThreads at a time together with their slots' page counts; a slot named
// again later in the list has nothing left to free by then.
__global__ void __launch_bounds__(kThreads)
dpam_free_kernel(jpt_dpam d, const int32_t* slots, int n_req, int slot_imm) {
  __shared__ int s_slot[kThreads], s_n[kThreads];
  const int head = d.state[0];
  int count = d.state[1];
  for (int r0 = 0; r0 < n_req; r0 += kThreads) {
    __syncthreads();  // the previous batch is done, its page counts are written
    const int n_here = min(kThreads, n_req - r0);
    int slot = -1, n = 0;
    if (static_cast<int>(threadIdx.x) < n_here) {
      slot = slots ? slots[r0 + threadIdx.x] : slot_imm;
      if (slot >= 0 && slot < d.batch) n = d.n_alloc[slot];
    }
    s_slot[threadIdx.x] = slot;
    __syncthreads();
    for (int j = 0; j < static_cast<int>(threadIdx.x) && j < n_here; ++j)
      if (s_slot[j] == slot) n = 0;
    s_n[threadIdx.x] = n;
    __syncthreads();
    for (int j = 0; j < n_here; ++j) {
      const int sl = s_slot[j];
      if (sl < 0 || sl >= d.batch) {
        if (threadIdx.x == 0) raise(d, JPT_DPAM_BADARG);
        continue;
      }
      int32_t* row = d.page_indices + static_cast<int64_t>(sl) * d.max_pages;
      // never more than the ring has room for
      const int m = min(max(s_n[j], 0), min(d.max_pages, d.total_pages - count));
      const int tail = (head + count) % d.total_pages;
      // a thread reads the cells it resets: no barrier between the two
      for (int i = threadIdx.x; i < d.max_pages; i += kThreads) {
        if (i < m) d.ring[(tail + i) % d.total_pages] = row[i];
        row[i] = d.total_pages - 1;
      }
      if (threadIdx.x == 0) {
        d.n_alloc[sl] = 0;
        d.lengths[sl] = 0;
      }
      count += m;
    }
  }
  if (threadIdx.x == 0) d.state[1] = count;
}

// fill_new_pages (:55-64) followed by get_page_token_indices (:145-177) on the
// same lens.  A slot whose length sits on a page boundary takes the next free
// page, slots in ascending order; then every slot with lens != 0 gets a column
// (page of its new token, j * page_size + token offset, slot) in
// update_indices, j counting the active slots in ascending order, and
// lengths = lens + 1 (0 where lens == 0).
__global__ void __launch_bounds__(kThreads)
dpam_decode_step_kernel(jpt_dpam d, const int32_t* lens) {
  const int head = d.state[0], count = d.state[1];
  const int ps = d.page_size;
  int popped = 0, active = 0;  // running totals over the slots handled so far
  for (int base = 0; base < d.batch; base += kThreads) {
    const int b = base + threadIdx.x;
    int len = b < d.batch ? lens[b] : 0;
    if (len < 0) {
      raise(d, JPT_DPAM_BADARG);
      len = 0;
    }
    const int p = len / ps;  // page that receives the token at position len
    const bool inside = p < d.max_pages;
    if (len > 0 && !inside) raise(d, JPT_DPAM_OVERFLOW);
    const bool wants = len > 0 && len % ps == 0 && inside;
    int n_wants, n_active;
    const int rank = popped + block_exclusive_scan(wants ? 1 : 0, &n_wants);
    const int j = active + block_exclusive_scan(len > 0 ? 1 : 0, &n_active);
    int32_t* row = d.page_indices + static_cast<int64_t>(b < d.batch ? b : 0) * d.max_pages;
    // page = -1: the step's token of this slot has no page (a request that
    // failed now or in an earlier step); the appends skip such a column, the
    // table cell says so too, and the slot's length stays where it was
    int page = -1;
    if (len > 0 && inside) page = row[p];
    if (wants) {
      if (rank < count) {
        page = d.ring[(head + rank) % d.total_pages];
        row[p] = page;
        d.n_alloc[b] = p + 1;
      } else {
        raise(d, JPT_DPAM_NOPAGES);
        page = -1;
        row[p] = -1;
      }
    }
    if (page >= d.total_pages) page = -1;
    if (b < d.batch) {
      d.lengths[b] = len > 0 && page >= 0 ? len + 1 : len;
      if (len > 0) {
        d.update_indices[j] = page;
        d.update_indices[d.batch + j] = j * ps + len % ps;
        d.update_indices[2 * d.batch + j] = b;
      }
    }
    popped += n_wants;
    active += n_active;
  }
  if (threadIdx.x == 0) {
    const int given = min(popped, count);
    d.state[0] = (head + given) % d.total_pages;
    d.state[1] = count - given;
    d.state[3] = active;
  }
}

template <typename T>
__global__ void __launch_bounds__(kThreads)
decode_advance_kernel(T* mask, int64_t mask_stride, int32_t* input_pos, int32_t* lens, int batch, int seq,
                      int ring_buffer, int current_position, int update_mask, int advance) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= batch) return;
  const int pos = input_pos[b];
  if (update_mask && mask) {
    const int at = ring_buffer ? current_position : pos;
    if (at >= 0 && at < seq) mask[b * mask_stride + at] = static_cast<T>(0);
  }
  if (advance) {
    // engine.py:800-812: `x + 1 % cache_len` is x + 1
    input_pos[b] = ring_buffer ? pos + 1 : (pos == 0 ? 0 : pos + 1);
    if (lens) {
      const int n = lens[b];
      lens[b] = ring_buffer ? n + 1 : (n == 0 ? 0 : n + 1);
    }
  }
}

// One thread per cell (slot b, block i) of the reference's block-index tables:
// the block the ring-aware ragged kernel of the reference would work on from
// that grid cell (engine.py:674-729).  end = (start + input_pos) % cache_len.
__global__ void __launch_bounds__(kThreads)
ragged_block_indices_kernel(const int32_t* start, const int32_t* input_pos, int batch, int cache_len, int bk,
                            int num_bk, int32_t* b_next, int32_t* i_next) {
  const int cell = blockIdx.x * blockDim.x + threadIdx.x;
  if (cell >= batch * num_bk) return;
  const int b = cell / num_bk, i = cell - b * num_bk;
  const int s = start[b];
  const int e = static_cast<int>((static_cast<int64_t>(s) + input_pos[b]) % cache_len);
  const bool last = b == batch - 1;
  // where a finished slot hands over: block 0 of the next slot; the last slot
  // stays on its own last block that can hold a live position
  const int hand_b = last ? b : b + 1;
  const int hand_i = last ? (s < e ? (e - 1) / bk : (cache_len - 1) / bk) : 0;
  int nb = b, ni = i;
  if (s < e) {
    if (i * bk >= e) { nb = hand_b; ni = hand_i; }
    if ((i + 1) * bk <= s) ni = s / bk;
  } else if (s == e) {
    nb = hand_b;
    ni = hand_i;
  } else if (i * bk >= e && (i + 1) * bk <= s) {
    ni = s / bk;
  }
  b_next[cell] = nb;
  i_next[cell] = ni;
}

int32_t check_dpam(const jpt_dpam* pam) {
  JPT_REQUIRE(pam != nullptr, "pam is NULL");
  JPT_REQUIRE(pam->state && pam->ring && pam->page_indices && pam->lengths && pam->n_alloc && pam->update_indices,
              "jpt_dpam has a NULL array");
  JPT_REQUIRE(pam->batch > 0 && pam->total_pages > 0 && pam->page_size > 0 && pam->max_pages > 0,
              "batch, total_pages, page_size, max_pages must be positive");
  return JPT_OK;
}

}  // namespace
}  // namespace jpt

extern "C" {

int32_t jpt_dpam_init(const jpt_dpam* pam, const int32_t* free_order, void* stream) {
  using namespace jpt;
  int32_t st = check_dpam(pam);
  if (st != JPT_OK) return st;
  const int64_t most = std::max<int64_t>(pam->total_pages, static_cast<int64_t>(pam->batch) * pam->max_pages);
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((most + kThreads - 1) / kThreads, 1024));
  hipLaunchKernelGGL(dpam_init_kernel, dim3(blocks), dim3(kThreads), 0, static_cast<hipStream_t>(stream), *pam, free_order);
  return launch_status("dpam_init_kernel");
}

int32_t jpt_dpam_reserve_insert(const jpt_dpam* pam, const int32_t* slots, const int32_t* seq_lens,
                                int32_t n_req, int32_t slot, int32_t seq_len, void* stream) {
  using namespace jpt;
  int32_t st = check_dpam(pam);
  if (st != JPT_OK) return st;
  JPT_REQUIRE((slots == nullptr) == (seq_lens == nullptr), "slots and seq_lens go together");
  JPT_REQUIRE(n_req >= 0 && (slots != nullptr || n_req <= 1), "n_req must be 0 or 1 without request arrays");
  if (n_req == 0) return JPT_OK;
  if (!slots) {
    JPT_REQUIRE(slot >= 0 && slot < pam->batch, "slot %d out of range", slot);
    JPT_REQUIRE(seq_len >= 0, "negative seq_len");
  }
  hipLaunchKernelGGL(dpam_reserve_insert_kernel, dim3(1), dim3(kThreads), 0, static_cast<hipStream_t>(stream), *pam,
                     slots, seq_lens, n_req, slot, seq_len);
  return launch_status("dpam_reserve_insert_kernel");
}

int32_t jpt_dpam_free(const jpt_dpam* pam, const int32_t* slots, int32_t n_req, int32_t slot, void* stream) {
  using namespace jpt;
  int32_t st = check_dpam(pam);
  if (st != JPT_OK) return st;
  JPT_REQUIRE(n_req >= 0 && (slots != nullptr || n_req <= 1), "n_req must be 0 or 1 without a slot array");
  if (n_req == 0) return JPT_OK;
  if (!slots) JPT_REQUIRE(slot >= 0 && slot < pam->batch, "slot %d out of range", slot);
  hipLaunchKernelGGL(dpam_free_kernel, dim3(1), dim3(kThreads), 0, static_cast<hipStream_t>(stream), *pam, slots,
                     n_req, slot);
  return launch_status("dpam_free_kernel");
}

int32_t jpt_dpam_decode_step(const jpt_dpam* pam, const int32_t* lens, void* stream) {
  using namespace jpt;
  int32_t st = check_dpam(pam);
  if (st != JPT_OK) return st;
  JPT_REQUIRE(lens != nullptr, "lens is NULL");
  hipLaunchKernelGGL(dpam_decode_step_kernel, dim3(1), dim3(kThreads), 0, static_cast<hipStream_t>(stream), *pam, lens);
  return launch_status("dpam_decode_step_kernel");
}

int32_t jpt_decode_advance(void* mask, int32_t mask_dtype, int64_t mask_stride, int32_t* input_pos,
                           int32_t* lens, int32_t batch, int32_t seq, int32_t ring_buffer,
                           int32_t current_position, int32_t update_mask, int32_t advance, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(input_pos != nullptr, "input_pos is NULL");
  JPT_REQUIRE(batch > 0 && seq > 0, "batch and seq must be positive");
  if (mask) {
    JPT_REQUIRE(mask_dtype == JPT_F32 || mask_dtype == JPT_BF16, "mask_dtype must be f32 or bf16");
    JPT_REQUIRE(mask_stride >= seq, "mask rows overlap");
  }
  const dim3 grid((batch + kThreads - 1) / kThreads);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (mask_dtype == JPT_BF16)
    hipLaunchKernelGGL(decode_advance_kernel<uint16_t>, grid, dim3(kThreads), 0, s, static_cast<uint16_t*>(mask),
                       mask_stride, input_pos, lens, batch, seq, ring_buffer, current_position, update_mask, advance);
  else
    hipLaunchKernelGGL(decode_advance_kernel<float>, grid, dim3(kThreads), 0, s, static_cast<float*>(mask),
                       mask_stride, input_pos, lens, batch, seq, ring_buffer, current_position, update_mask, advance);
  return launch_status("decode_advance_kernel");
}

int32_t jpt_ragged_block_indices(const int32_t* start, const int32_t* input_pos, int32_t batch, int32_t cache_len,
                                 int32_t block_size, int32_t* b_next, int32_t* i_next, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(start && input_pos && b_next && i_next, "NULL argument");
  JPT_REQUIRE(batch > 0 && cache_len > 0 && block_size > 0, "batch, cache_len and block_size must be positive");
  JPT_REQUIRE(cache_len % block_size == 0, "cache_len must be a multiple of block_size");
  const int num_bk = cache_len / block_size;
  JPT_REQUIRE(static_cast<int64_t>(batch) * num_bk <= INT32_MAX, "table too large");
  const dim3 grid((batch * num_bk + kThreads - 1) / kThreads);
  hipLaunchKernelGGL(ragged_block_indices_kernel, grid, dim3(kThreads), 0, static_cast<hipStream_t>(stream), start,
                     input_pos, batch, cache_len, block_size, num_bk, b_next, i_next);
  return launch_status("ragged_block_indices_kernel");
}

}  // extern "C"
