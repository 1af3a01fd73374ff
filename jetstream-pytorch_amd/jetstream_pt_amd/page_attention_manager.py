"""PageAttentionManager: host page allocator + the kernels that consume its tables.

Same constructor and methods as the reference class
(jetstream_pt/page_attention_manager.py:11-222).  The free list, the page
table and the lengths live in the C++ allocator of libjpt_mi355.so;
`page_indices` and `lengths` are numpy views of that memory, so
`reserve_pages_insert` returns a view of the table row exactly like the
reference does.  Tensor arguments are torch tensors on the ROCm device.
"""

import ctypes
from typing import List, Tuple

import numpy as np
import torch

from . import _ffi


class PageAttentionManager:

  def __init__(self, batch_size: int, paged_attention_total_num_pages: int,
               paged_attention_page_size: int, max_pages_per_sequence: int,
               *, free_list_order=None):
    self.batch_size = batch_size
    self.paged_attention_total_num_pages = paged_attention_total_num_pages
    self.paged_attention_page_size = paged_attention_page_size
    self.max_pages_per_sequence = max_pages_per_sequence
    order = None
    if free_list_order is not None:
      arr = np.ascontiguousarray(np.asarray(free_list_order, dtype=np.int32))
      if arr.shape != (paged_attention_total_num_pages,):
        raise ValueError("free_list_order must list every page id once")
      order = arr.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
    handle = ctypes.c_void_p()
    _ffi.check(_ffi.lib.jpt_pam_create(
        batch_size, paged_attention_total_num_pages, paged_attention_page_size,
        max_pages_per_sequence, order, ctypes.byref(handle)))
    self._handle = handle
    pi, ln = ctypes.POINTER(ctypes.c_int32)(), ctypes.POINTER(ctypes.c_int32)()
    _ffi.check(_ffi.lib.jpt_pam_tables(handle, ctypes.byref(pi), ctypes.byref(ln)))
    self.page_indices = np.ctypeslib.as_array(pi, shape=(batch_size, max_pages_per_sequence))
    self._lengths = np.ctypeslib.as_array(ln, shape=(batch_size,))
    self._scratch = np.empty(3 * batch_size, dtype=np.int32)
    self._device_tables = None

  def __del__(self, _destroy=_ffi.lib.jpt_pam_destroy):
    handle, self._handle = getattr(self, "_handle", None), None
    if handle:
      _destroy(handle)

  @property
  def lengths(self):
    return self._lengths

  @lengths.setter
  def lengths(self, value):
    # the reference rebinds `lengths` (page_attention_manager.py:167); here the
    # storage belongs to the allocator, so assignment copies into it
    self._lengths[:] = np.asarray(value, dtype=np.int32)
    self._device_tables = None

  @staticmethod
  def _i32(a):
    arr = np.ascontiguousarray(np.asarray(a, dtype=np.int32).reshape(-1))
    return arr, arr.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))

  # pylint: disable-next=all
  def reserve_pages_insert(self, slot: int, seq_len: int):
    n = ctypes.c_int32()
    _ffi.check(_ffi.lib.jpt_pam_reserve_insert(self._handle, int(slot), int(seq_len), ctypes.byref(n)))
    self._device_tables = None
    return n.value, self.page_indices[slot, : n.value]

  # pylint: disable-next=all
  def reserve_pages_decode(self, slot: int, seq_len: int):
    _ffi.check(_ffi.lib.jpt_pam_reserve_decode(self._handle, int(slot), int(seq_len)))
    self._device_tables = None

  # pylint: disable-next=all
  def fill_new_pages(self, lens):
    arr, p = self._i32(lens)
    if arr.size != self.batch_size:
      raise ValueError(f"lens must have {self.batch_size} entries")
    _ffi.check(_ffi.lib.jpt_pam_fill_new_pages(self._handle, p))
    self._device_tables = None

  # pylint: disable-next=all
  def get_page_token_indices(self, lens):
    arr, p = self._i32(lens)
    if arr.size != self.batch_size:
      raise ValueError(f"lens must have {self.batch_size} entries")
    n = ctypes.c_int32()
    out = self._scratch.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
    _ffi.check(_ffi.lib.jpt_pam_page_token_indices(self._handle, p, out, ctypes.byref(n)))
    self._device_tables = None
    return self._scratch[: 3 * n.value].reshape(3, n.value).copy()

  # pylint: disable-next=all
  def free_pages_resource(self, slot):
    _ffi.check(_ffi.lib.jpt_pam_free(self._handle, int(slot)))
    self._device_tables = None
    return None

  free_pages = free_pages_resource

  def unused_page_ids(self):
    """The free list in hand-out order (for tests and accounting)."""
    n = _ffi.lib.jpt_pam_free_count(self._handle, None)
    out = np.empty(max(n, 1), dtype=np.int32)
    _ffi.lib.jpt_pam_free_count(self._handle, out.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)))
    return out[:n]

  def device_tables(self, device):
    """(lengths, page_indices) as int32 device tensors, re-uploaded only after
    the allocator state changed."""
    cached = self._device_tables
    if cached is None or cached[0].device != torch.device(device):
      cached = (torch.from_numpy(self._lengths.copy()).to(device),
                torch.from_numpy(self.page_indices.copy()).to(device))
      self._device_tables = cached
    return cached

  def insert_prefill_cache(self, prefill_caches: List[Tuple[torch.Tensor, torch.Tensor]],
                           decode_caches: List[Tuple[torch.Tensor, torch.Tensor]],
                           update_indexes, tep_kv=None, sharding=None):
    """Copies each layer's prefill K/V (1, heads, seq, dim) into the pages
    `update_indexes`, zero-filling the tail of the last page.  In place; returns
    the decode caches.  `tep_kv` and `sharding` are accepted and unused (the
    kernel needs no padded staging buffer)."""
    if not decode_caches:
      return decode_caches
    device = decode_caches[0][0].device
    ids = _ffi.as_i32(update_indexes, device)
    for (k, v), (pk, pv) in zip(prefill_caches, decode_caches):
      _ffi.dev(pk, "decode cache"), _ffi.dev(pv, "decode cache")
      heads, total, ps, dim = pk.shape
      k = _ffi.dev(k.to(pk.dtype).contiguous(), "prefill k")
      v = _ffi.dev(v.to(pv.dtype).contiguous(), "prefill v")
      if k.shape[0] != 1 or k.shape[1] != heads or k.shape[3] != dim:
        raise ValueError(f"prefill cache {tuple(k.shape)} does not match pages {tuple(pk.shape)}")
      _ffi.check(_ffi.lib.jpt_paged_insert(
          _ffi.ptr(pk), _ffi.ptr(pv), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(ids), ids.numel(),
          k.shape[2], heads, total, ps, dim * pk.element_size(), _ffi.stream()))
    return decode_caches

  # pylint: disable-next=all
  def get_compress_kv_cache(self, decode_caches, slot: int):
    lens, indices = int(self._lengths[slot]), self.page_indices[slot]
    return [(self._compress_cache(k, lens, indices), self._compress_cache(v, lens, indices))
            for k, v in decode_caches]

  def _compress_cache(self, cache: torch.Tensor, lens: int, indices):
    _ffi.dev(cache, "cache")
    heads, total, ps, dim = cache.shape
    row = _ffi.as_i32(indices, cache.device)
    out = torch.empty((heads, lens, dim), dtype=cache.dtype, device=cache.device)
    if lens == 0:
      return out
    _ffi.check(_ffi.lib.jpt_paged_gather(
        _ffi.ptr(out), _ffi.ptr(cache), _ffi.ptr(row), lens, heads, total, ps,
        dim * cache.element_size(), _ffi.stream()))
    return out
