"""PageAttentionManager: page allocator + the kernels that consume its tables.

Same constructor and methods as the reference class
(jetstream_pt/page_attention_manager.py:11-222).  The free list, the page
table and the lengths live in the C++ allocator of libjpt_mi355.so;
`page_indices` and `lengths` are numpy views of that memory, so
`reserve_pages_insert` returns a view of the table row exactly like the
reference does.  Tensor arguments are torch tensors on the ROCm device.

DevicePageAttentionManager keeps the same state in HBM and runs every method as
a small kernel: nothing crosses PCIe during a decode step, and the step can be
captured in a HIP graph.  Same hand-out order and tables as the host class.
"""

import ctypes
import queue
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
    self._touch()

  def _touch(self):
    """The tables changed: device copies and split plans made from them are stale."""
    self._device_tables = None
    self._version = getattr(self, "_version", 0) + 1

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
    self._touch()

  @staticmethod
  def _i32(a):
    arr = np.ascontiguousarray(np.asarray(a, dtype=np.int32).reshape(-1))
    return arr, arr.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))

  # pylint: disable-next=all
  def reserve_pages_insert(self, slot: int, seq_len: int):
    n = ctypes.c_int32()
    _ffi.check(_ffi.lib.jpt_pam_reserve_insert(self._handle, int(slot), int(seq_len), ctypes.byref(n)))
    self._touch()
    return n.value, self.page_indices[slot, : n.value]

  # pylint: disable-next=all
  def reserve_pages_decode(self, slot: int, seq_len: int):
    _ffi.check(_ffi.lib.jpt_pam_reserve_decode(self._handle, int(slot), int(seq_len)))
    self._touch()

  # pylint: disable-next=all
  def fill_new_pages(self, lens):
    arr, p = self._i32(lens)
    if arr.size != self.batch_size:
      raise ValueError(f"lens must have {self.batch_size} entries")
    _ffi.check(_ffi.lib.jpt_pam_fill_new_pages(self._handle, p))
    self._touch()

  # pylint: disable-next=all
  def get_page_token_indices(self, lens):
    arr, p = self._i32(lens)
    if arr.size != self.batch_size:
      raise ValueError(f"lens must have {self.batch_size} entries")
    n = ctypes.c_int32()
    out = self._scratch.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
    _ffi.check(_ffi.lib.jpt_pam_page_token_indices(self._handle, p, out, ctypes.byref(n)))
    self._touch()
    return self._scratch[: 3 * n.value].reshape(3, n.value).copy()

  # pylint: disable-next=all
  def free_pages_resource(self, slot):
    _ffi.check(_ffi.lib.jpt_pam_free(self._handle, int(slot)))
    self._touch()
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
    if len(decode_caches) > 1:  # all layers in one launch where their shapes allow
      from . import insert as _insert
      if _insert.insert_prefix_pages_copy(prefill_caches, decode_caches, ids):
        return decode_caches
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
        _ffi.ptr(out), _ffi.ptr(cache), _ffi.ptr(row), row.numel(), lens, heads, total, ps,
        dim * cache.element_size(), _ffi.stream()))
    return out


class DeviceTokenIndices:
  """What get_page_token_indices returns when the tables live on the device:
  `indices` (3, stride) int32 with the first `n_active[0]` columns valid,
  `n_active` a one-element int32 device tensor.  The paged caches' update()
  takes it where it takes the reference's (3, n_active) array."""

  def __init__(self, indices, n_active):
    self.indices, self.n_active, self.stride = indices, n_active, indices.shape[1]

  def to_host(self):
    """(3, n_active) numpy array, as the reference returns it (synchronises)."""
    n = int(self.n_active.item())
    return self.indices[:, :n].cpu().numpy()


class DevicePageAttentionManager(PageAttentionManager):
  """PageAttentionManager with free list, page table and lengths on the device.

  Methods enqueue one-workgroup kernels on the current stream and return at
  once.  Differences a caller sees:
    * `page_indices` and `lengths` are int32 device tensors (views of the
      allocator's memory, so `reserve_pages_insert` still returns a view of
      the table row);
    * `fill_new_pages(lens)` takes the device tensor of per-slot lengths and
      also prepares what `get_page_token_indices(lens)` returns, a
      DeviceTokenIndices;
    * a kernel cannot raise: a request that cannot be served is skipped and
      remembered; `check()` (synchronises) raises queue.Empty / IndexError /
      ValueError for it like the host class does at once.  Until then
      `reserve_pages_insert` has returned the view of the row it would have
      filled, and a decode step has dropped the token of a slot it found no
      page for (page id -1 in its index column and table cell; no other
      slot's page is touched).
  """

  # pylint: disable-next=super-init-not-called
  def __init__(self, batch_size: int, paged_attention_total_num_pages: int,
               paged_attention_page_size: int, max_pages_per_sequence: int,
               *, device="cuda", free_list_order=None):
    self.batch_size = batch_size
    self.paged_attention_total_num_pages = paged_attention_total_num_pages
    self.paged_attention_page_size = paged_attention_page_size
    self.max_pages_per_sequence = max_pages_per_sequence
    self._handle = None
    b, total, mp = batch_size, paged_attention_total_num_pages, max_pages_per_sequence
    if min(b, total, paged_attention_page_size, mp) <= 0:
      raise ValueError("batch, total pages, page size and pages per sequence must be positive")
    sizes = [4, total, b * mp, b, b, 3 * b]
    offs = [0]
    for n in sizes:
      offs.append(offs[-1] + (n + 63) // 64 * 64)  # 256-byte aligned pieces
    self._mem = torch.zeros(offs[-1], dtype=torch.int32, device=device)
    piece = lambda i: self._mem[offs[i]: offs[i] + sizes[i]]
    self._state, self._ring = piece(0), piece(1)
    self.page_indices = piece(2).view(b, mp)
    self._lengths, self._n_alloc = piece(3), piece(4)
    self._update_indices = piece(5).view(3, b)
    self._c = _ffi.Dpam(
        state=_ffi.ptr(self._state), ring=_ffi.ptr(self._ring), page_indices=_ffi.ptr(self.page_indices),
        lengths=_ffi.ptr(self._lengths), n_alloc=_ffi.ptr(self._n_alloc),
        update_indices=_ffi.ptr(self._update_indices), batch=b, total_pages=total,
        page_size=paged_attention_page_size, max_pages=mp)
    order = None
    if free_list_order is not None:
      arr = np.ascontiguousarray(np.asarray(free_list_order, dtype=np.int32))
      if arr.shape != (total,) or not np.array_equal(np.sort(arr), np.arange(total, dtype=np.int32)):
        raise ValueError("free_list_order must list every page id once")
      order = torch.from_numpy(arr).to(device)
    _ffi.check(_ffi.lib.jpt_dpam_init(self._c, _ffi.ptr(order), _ffi.stream()))
    self._keep = order  # read by the enqueued kernel
    self._token_indices = DeviceTokenIndices(self._update_indices, self._state[3:4])
    self._stepped = False
    self.step_lens = None
    self._version = 1  # bumped by every launch that changes `lengths`

  def __del__(self):
    return

  @property
  def lengths(self):
    return self._lengths

  @lengths.setter
  def lengths(self, value):
    self._lengths.copy_(torch.as_tensor(value, dtype=torch.int32))
    self._version += 1

  def _req(self, x):
    return _ffi.as_i32(x, self._mem.device)

  # pylint: disable-next=all
  def reserve_pages_insert(self, slot: int, seq_len: int):
    slot, seq_len = int(slot), int(seq_len)
    _ffi.check(_ffi.lib.jpt_dpam_reserve_insert(self._c, None, None, 1, slot, seq_len, _ffi.stream()))
    self._version += 1
    ps = self.paged_attention_page_size
    n = (seq_len + ps - 1) // ps
    return n, self.page_indices[slot, :n]

  def reserve_pages_insert_many(self, slots, seq_lens):
    """reserve_pages_insert for several slots, in the order given, in one launch;
    slots and seq_lens may be device tensors (no host copy)."""
    slots, seq_lens = self._req(slots), self._req(seq_lens)
    if slots.numel() != seq_lens.numel():
      raise ValueError("slots and seq_lens differ in length")
    _ffi.check(_ffi.lib.jpt_dpam_reserve_insert(
        self._c, _ffi.ptr(slots), _ffi.ptr(seq_lens), slots.numel(), 0, 0, _ffi.stream()))
    self._keep = (slots, seq_lens)
    self._version += 1

  # pylint: disable-next=all
  def reserve_pages_decode(self, slot: int, seq_len: int):
    raise NotImplementedError("the device allocator serves all slots of a step at once: fill_new_pages(lens)")

  # pylint: disable-next=all
  def fill_new_pages(self, lens):
    lens = _ffi.dev(lens, "lens")
    if lens.dtype != torch.int32 or lens.numel() != self.batch_size:
      raise ValueError(f"lens must be an int32 device tensor of {self.batch_size} entries")
    _ffi.check(_ffi.lib.jpt_dpam_decode_step(self._c, _ffi.ptr(lens), _ffi.stream()))
    self._stepped = True
    self._version += 1
    # the lengths before the step's token, for an attention launch that appends
    # the token itself; valid until the caller advances `lens`
    self.step_lens = lens

  # pylint: disable-next=all
  def get_page_token_indices(self, lens):
    if not self._stepped:
      raise RuntimeError("call fill_new_pages(lens) first: on the device both run as one kernel")
    self._stepped = False
    return self._token_indices

  def decode_step(self, lens):
    """fill_new_pages(lens) + get_page_token_indices(lens)."""
    self.fill_new_pages(lens)
    return self.get_page_token_indices(lens)

  # pylint: disable-next=all
  def free_pages_resource(self, slot):
    _ffi.check(_ffi.lib.jpt_dpam_free(self._c, None, 1, int(slot), _ffi.stream()))
    self._version += 1
    return None

  free_pages = free_pages_resource

  def free_pages_resource_many(self, slots):
    slots = self._req(slots)
    _ffi.check(_ffi.lib.jpt_dpam_free(self._c, _ffi.ptr(slots), slots.numel(), 0, _ffi.stream()))
    self._keep = slots
    self._version += 1

  def status(self):
    """Failure bits recorded by the kernels so far (synchronises)."""
    return int(self._state[2].item())

  def check(self):
    """Raises what the host class raises at once, for every request the kernels
    could not serve since the last check (synchronises); the record is cleared,
    so the next check reports new failures only.  A decode step whose page
    request failed has dropped that slot's token: nothing was written for it."""
    bits = self.status()
    if bits:
      self._state[2:3].zero_()
    if bits & _ffi.DPAM_NOPAGES:
      raise queue.Empty("the device free list ran out of pages")
    if bits & _ffi.DPAM_OVERFLOW:
      raise IndexError("a slot needed more pages than max_pages_per_sequence")
    if bits & _ffi.DPAM_BADARG:
      raise ValueError("a slot id or length given to the device allocator was out of range")

  def unused_page_ids(self):
    """The free list in hand-out order (synchronises; for tests and accounting)."""
    head, count = (int(x) for x in self._state[:2].tolist())
    ring = self._ring.cpu().numpy()
    total = self.paged_attention_total_num_pages
    return ring[(head + np.arange(count)) % total]

  def device_tables(self, device):
    return self._lengths, self.page_indices

  # pylint: disable-next=all
  def get_compress_kv_cache(self, decode_caches, slot: int):
    lens, indices = int(self._lengths[slot].item()), self.page_indices[slot]
    return [(self._compress_cache(k, lens, indices), self._compress_cache(v, lens, indices))
            for k, v in decode_caches]
