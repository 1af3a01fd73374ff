// Host page allocator behind PageAttentionManager
// (reference: jetstream_pt/page_attention_manager.py:21-64, :145-177, :214-222).
//
// A FIFO ring of page ids plus the (batch, max_pages) page table and the
// per-slot lengths, all in host memory owned by the handle.  The Python class
// wraps page table and lengths as numpy views, which gives callers the same
// aliasing the reference has (reserve_pages_insert returns a view of the row).
#include <mutex>
#include <new>
#include <vector>

#include "common.h"

struct jpt_pam {
  int32_t batch, total_pages, page_size, max_pages;
  std::vector<int32_t> ring;  // free list: `count` ids starting at `head`
  int64_t head = 0, count = 0;
  std::vector<int32_t> page_indices;  // batch * max_pages
  std::vector<int32_t> lengths;       // batch
  std::vector<int32_t> n_alloc;       // pages this slot was handed
  std::mutex mu;

  bool pop(int32_t* id) {
    if (count == 0) return false;
    *id = ring[head];
    head = (head + 1) % total_pages;
    --count;
    return true;
  }
  void push(int32_t id) {
    ring[(head + count) % total_pages] = id;
    ++count;
  }
};

namespace {

int32_t reserve_decode_locked(jpt_pam* p, int32_t slot, int32_t seq_len) {
  // page_attention_manager.py:55-59
  if (seq_len <= 0 || seq_len % p->page_size != 0) return JPT_OK;
  int32_t n = seq_len / p->page_size;
  if (n >= p->max_pages)
    return jpt::fail(JPT_E_PAGE_OVERFLOW,
                     "slot %d at length %d needs page %d of at most %d", slot,
                     seq_len, n + 1, p->max_pages);
  int32_t id;
  if (!p->pop(&id))
    return jpt::fail(JPT_E_NOPAGES, "free list empty (decode, slot %d)", slot);
  p->page_indices[static_cast<size_t>(slot) * p->max_pages + n] = id;
  p->n_alloc[slot] = n + 1;
  return JPT_OK;
}

}  // namespace

extern "C" {

int32_t jpt_pam_create(int32_t batch, int32_t total_pages, int32_t page_size,
                       int32_t max_pages, const int32_t* free_order,
                       jpt_pam** out) {
  JPT_REQUIRE(out != nullptr, "out is NULL");
  JPT_REQUIRE(batch > 0 && total_pages > 0 && page_size > 0 && max_pages > 0,
              "batch, total_pages, page_size, max_pages must be positive");
  if (free_order) {
    std::vector<char> seen(total_pages, 0);
    for (int32_t i = 0; i < total_pages; ++i) {
      int32_t id = free_order[i];
      JPT_REQUIRE(id >= 0 && id < total_pages && !seen[id],
                  "free_order is not a permutation of 0..%d", total_pages - 1);
      seen[id] = 1;
    }
  }
  jpt_pam* p = new (std::nothrow) jpt_pam;
  JPT_REQUIRE(p != nullptr, "out of host memory");
  p->batch = batch;
  p->total_pages = total_pages;
  p->page_size = page_size;
  p->max_pages = max_pages;
  p->ring.resize(total_pages);
  for (int32_t i = 0; i < total_pages; ++i)
    p->ring[i] = free_order ? free_order[i] : i;  // :38-39
  p->count = total_pages;
  // :30-35: the sentinel is the last page id, which is itself allocatable
  p->page_indices.assign(static_cast<size_t>(batch) * max_pages, total_pages - 1);
  p->lengths.assign(batch, 0);
  p->n_alloc.assign(batch, 0);
  *out = p;
  return JPT_OK;
}

void jpt_pam_destroy(jpt_pam* pam) { delete pam; }

int32_t jpt_pam_tables(jpt_pam* pam, int32_t** page_indices, int32_t** lengths) {
  JPT_REQUIRE(pam != nullptr, "pam is NULL");
  if (page_indices) *page_indices = pam->page_indices.data();
  if (lengths) *lengths = pam->lengths.data();
  return JPT_OK;
}

int32_t jpt_pam_reserve_insert(jpt_pam* pam, int32_t slot, int32_t seq_len,
                               int32_t* num_pages) {
  JPT_REQUIRE(pam != nullptr, "pam is NULL");
  JPT_REQUIRE(slot >= 0 && slot < pam->batch, "slot %d out of range", slot);
  JPT_REQUIRE(seq_len >= 0, "negative seq_len");
  std::lock_guard<std::mutex> lock(pam->mu);
  // :42-52
  int32_t n = (seq_len + pam->page_size - 1) / pam->page_size;
  if (n > pam->max_pages)
    return jpt::fail(JPT_E_PAGE_OVERFLOW, "%d tokens need %d pages, row holds %d",
                     seq_len, n, pam->max_pages);
  if (n > pam->count)
    return jpt::fail(JPT_E_NOPAGES, "need %d pages, %lld free", n,
                     static_cast<long long>(pam->count));
  pam->lengths[slot] = seq_len;
  int32_t* row = &pam->page_indices[static_cast<size_t>(slot) * pam->max_pages];
  for (int32_t i = 0; i < n; ++i) pam->pop(&row[i]);
  pam->n_alloc[slot] = n;
  if (num_pages) *num_pages = n;
  return JPT_OK;
}

int32_t jpt_pam_reserve_decode(jpt_pam* pam, int32_t slot, int32_t seq_len) {
  JPT_REQUIRE(pam != nullptr, "pam is NULL");
  JPT_REQUIRE(slot >= 0 && slot < pam->batch, "slot %d out of range", slot);
  std::lock_guard<std::mutex> lock(pam->mu);
  return reserve_decode_locked(pam, slot, seq_len);
}

int32_t jpt_pam_fill_new_pages(jpt_pam* pam, const int32_t* lens) {
  JPT_REQUIRE(pam != nullptr && lens != nullptr, "NULL argument");
  std::lock_guard<std::mutex> lock(pam->mu);
  for (int32_t slot = 0; slot < pam->batch; ++slot) {  // :62-64
    int32_t st = reserve_decode_locked(pam, slot, lens[slot]);
    if (st != JPT_OK) return st;
  }
  return JPT_OK;
}

int32_t jpt_pam_page_token_indices(jpt_pam* pam, const int32_t* lens,
                                   int32_t* out, int32_t* n_active) {
  JPT_REQUIRE(pam != nullptr && lens != nullptr && out != nullptr &&
                  n_active != nullptr, "NULL argument");
  std::lock_guard<std::mutex> lock(pam->mu);
  const int32_t ps = pam->page_size;
  int32_t n = 0;
  for (int32_t slot = 0; slot < pam->batch; ++slot) {
    if (lens[slot] == 0) continue;
    JPT_REQUIRE(lens[slot] > 0, "slot %d has negative length %d", slot, lens[slot]);
    if (lens[slot] / ps >= pam->max_pages)
      return jpt::fail(JPT_E_PAGE_OVERFLOW, "slot %d length %d outside the page table",
                       slot, lens[slot]);
    ++n;
  }
  // :145-177; rows are (page, offset + token, slot)
  int32_t j = 0;
  for (int32_t slot = 0; slot < pam->batch; ++slot) {
    int32_t len = lens[slot];
    if (len == 0) {
      pam->lengths[slot] = 0;
      continue;
    }
    out[j] = pam->page_indices[static_cast<size_t>(slot) * pam->max_pages + len / ps];
    out[n + j] = j * ps + len % ps;
    out[2 * n + j] = slot;
    pam->lengths[slot] = len + 1;  // :167
    ++j;
  }
  *n_active = n;
  return JPT_OK;
}

int32_t jpt_pam_free(jpt_pam* pam, int32_t slot) {
  JPT_REQUIRE(pam != nullptr, "pam is NULL");
  JPT_REQUIRE(slot >= 0 && slot < pam->batch, "slot %d out of range", slot);
  std::lock_guard<std::mutex> lock(pam->mu);
  int32_t* row = &pam->page_indices[static_cast<size_t>(slot) * pam->max_pages];
  for (int32_t i = 0; i < pam->n_alloc[slot]; ++i) pam->push(row[i]);
  for (int32_t i = 0; i < pam->max_pages; ++i) row[i] = pam->total_pages - 1;
  pam->n_alloc[slot] = 0;
  pam->lengths[slot] = 0;
  return JPT_OK;
}

int32_t jpt_pam_free_count(jpt_pam* pam, int32_t* out) {
  if (pam == nullptr) return jpt::fail(JPT_E_BADARG, "pam is NULL");
  std::lock_guard<std::mutex> lock(pam->mu);
  if (out)
    for (int64_t i = 0; i < pam->count; ++i)
      out[i] = pam->ring[(pam->head + i) % pam->total_pages];
  return static_cast<int32_t>(pam->count);
}

}  // extern "C"
