"""Host page allocator, restated with a deque and numpy (test infrastructure).

Follows jetstream_pt/page_attention_manager.py.  `free_pages_resource` is the
one method that does not follow the reference text: the reference version
raises AttributeError after pushing the whole table row, sentinel entries
included, back to the free list (page_attention_manager.py:214-222).  Here it
returns exactly the pages the slot was handed, in row order, resets the row
to the sentinel and the length to zero.
"""

import collections
import queue

import numpy as np
import torch


class PageAttentionManager:

  def __init__(self, batch_size, paged_attention_total_num_pages,
               paged_attention_page_size, max_pages_per_sequence,
               free_list_order=None):
    # page_attention_manager.py:28-39
    self.batch_size = batch_size
    self.total_num_pages = paged_attention_total_num_pages
    self.paged_attention_page_size = paged_attention_page_size
    self.max_pages_per_sequence = max_pages_per_sequence
    order = (range(paged_attention_total_num_pages)
             if free_list_order is None else free_list_order)
    self.unused_pages = collections.deque(int(i) for i in order)
    self.page_indices = np.full(
        (batch_size, max_pages_per_sequence),
        paged_attention_total_num_pages - 1, dtype=np.int32,
    )
    self.lengths = np.zeros(batch_size, dtype=np.int32)
    self._n_alloc = np.zeros(batch_size, dtype=np.int64)

  def _pop(self):
    if not self.unused_pages:
      raise queue.Empty  # Queue.get(block=False) on an empty queue
    return self.unused_pages.popleft()

  def reserve_pages_insert(self, slot, seq_len):
    """page_attention_manager.py:42-52."""
    ps = self.paged_attention_page_size
    self.lengths[slot] = seq_len
    num_pages = seq_len // ps if seq_len % ps == 0 else seq_len // ps + 1
    indices = [self._pop() for _ in range(num_pages)]
    self.page_indices[slot, :num_pages] = indices
    self._n_alloc[slot] = num_pages
    return num_pages, self.page_indices[slot, :num_pages]

  def reserve_pages_decode(self, slot, seq_len):
    """page_attention_manager.py:55-59."""
    ps = self.paged_attention_page_size
    if seq_len > 0 and seq_len % ps == 0:
      num_pages = seq_len // ps
      if num_pages >= self.max_pages_per_sequence:
        raise IndexError("sequence outgrew max_pages_per_sequence")
      self.page_indices[slot, num_pages] = self._pop()
      self._n_alloc[slot] = num_pages + 1

  def fill_new_pages(self, lens):
    """page_attention_manager.py:62-64."""
    for slot in range(self.batch_size):
      self.reserve_pages_decode(slot, int(lens[slot]))

  def get_page_token_indices(self, lens):
    """page_attention_manager.py:145-177."""
    ps = self.paged_attention_page_size
    lens = np.asarray(lens)
    pages, tokens, slots = [], [], []
    offset = 0
    for slot in range(self.batch_size):
      seq_len = int(lens[slot])
      if seq_len == 0:
        continue
      pages.append(self.page_indices[slot, seq_len // ps])
      tokens.append(offset + seq_len % ps)
      slots.append(slot)
      offset += ps
    self.lengths = np.where(lens == 0, 0, lens + 1)
    return np.stack((np.asarray(pages), np.asarray(tokens), np.asarray(slots)))

  def insert_prefill_cache(self, prefill_caches, decode_caches, update_indexes,
                           tep_kv=None, sharding=None):
    """page_attention_manager.py:83-142.

    prefill K/V (1, heads, seq, dim) -> zero-padded to whole pages ->
    (heads, n_pages, page_size, dim) -> written at pages `update_indexes`.
    """
    ps = self.paged_attention_page_size
    idx = torch.as_tensor(np.asarray(update_indexes), dtype=torch.int64)
    out = []
    for (k, v), (dk, dv) in zip(prefill_caches, decode_caches):
      for src, dst in ((k, dk), (v, dv)):
        src = src.squeeze(0)
        heads, seq, dim = src.shape
        padded = torch.zeros((heads, len(idx) * ps, dim), dtype=dst.dtype)
        padded[:, :seq, :] = src
        dst[:, idx, :, :] = padded.reshape(heads, -1, ps, dim)
      out.append((dk, dv))
    return out

  def _compress_cache(self, cache, lens, indices):
    """page_attention_manager.py:195-200."""
    head, _, _, dim = cache.shape
    idx = torch.as_tensor(np.asarray(indices), dtype=torch.int64)
    return cache[:, idx, :, :].reshape(head, -1, dim)[:, 0:int(lens), :]

  def get_compress_kv_cache(self, decode_caches, slot):
    """page_attention_manager.py:180-193."""
    lens, indices = self.lengths[slot], self.page_indices[slot]
    return [
        (self._compress_cache(k, lens, indices), self._compress_cache(v, lens, indices))
        for k, v in decode_caches
    ]

  def free_pages_resource(self, slot):
    n = int(self._n_alloc[slot])
    self.unused_pages.extend(int(p) for p in self.page_indices[slot, :n])
    self.page_indices[slot, :] = self.total_num_pages - 1
    self.lengths[slot] = 0
    self._n_alloc[slot] = 0
    return None

  free_pages = free_pages_resource
