"""Per-step decode-state bookkeeping on the device.

The reference's generate step (jetstream_pt/engine.py:774-817) unmasks each
slot's new position in the attention mask and advances `input_pos` and `lens`
with a handful of jnp ops; with paged attention it first pulls `input_pos` to
the host for the page allocator (:739-745).  Here both are one small launch on
device-resident int32 tensors, in place, so a whole decode step can be
enqueued (or captured in a HIP graph) without a host round trip.
"""

import torch

from . import _ffi


def _advance(mask, input_pos, lens, ring_buffer, current_position, update, advance):
  input_pos = _ffi.dev(input_pos, "input_pos")
  if input_pos.dtype != torch.int32:
    raise ValueError("input_pos must be an int32 device tensor (it is updated in place)")
  batch = input_pos.numel()
  mptr, mdt, stride, seq = None, _ffi.F32, 1, 1
  if mask is not None:
    if mask.dim() != 2 or mask.shape[0] != batch or mask.stride(1) != 1 or not mask.is_cuda:
      raise ValueError("mask must be a (batch, seq) device tensor with unit stride along seq")
    mptr, mdt, stride, seq = _ffi.ptr(mask), _ffi.dtype_code(mask.dtype), mask.stride(0), mask.shape[1]
  if lens is not None:
    lens = _ffi.dev(lens, "lens")
    if lens.dtype != torch.int32 or lens.numel() != batch:
      raise ValueError("lens must be an int32 device tensor with one entry per slot")
  _ffi.check(_ffi.lib.jpt_decode_advance(
      mptr, mdt, stride, _ffi.ptr(input_pos), _ffi.ptr(lens), batch, seq, int(bool(ring_buffer)),
      int(current_position), int(update), int(advance), _ffi.stream()))


def update_mask(mask, input_pos, *, ring_buffer=False, current_position=0):
  """mask[b, input_pos[b]] = 0, or mask[:, current_position] = 0 with a ring
  buffer (update_mask in generate_impl, engine.py:774-780); in place."""
  _advance(mask, input_pos, None, ring_buffer, current_position, True, False)
  return mask


def advance(input_pos, lens=None, *, ring_buffer=False):
  """input_pos and lens after a step: x == 0 ? 0 : x + 1, or x + 1 with a ring
  buffer (engine.py:800-812; `x + 1 % cache_len` there is x + 1); in place."""
  _advance(None, input_pos, lens, ring_buffer, 0, False, True)
  return input_pos, lens


def finish_step(mask, input_pos, lens=None, *, ring_buffer=False, current_position=0):
  """update_mask with the positions before the step, then advance: the lazy-update
  order of generate_impl, one launch."""
  _advance(mask, input_pos, lens, ring_buffer, current_position, True, True)
  return mask, input_pos, lens


def ragged_block_indices(start, input_pos, cache_len, block_size):
  """The reference's Engine.precompute_ragged_block_indices (engine.py:674-729)
  on device tensors: start, input_pos (batch) int32; returns (b_next, i_next),
  each (batch, cache_len // block_size) int32.  The attention entry points of
  this package do not read them (the reference's live kernel does not either);
  for callers whose decode state carries the tables."""
  start = _ffi.dev(start, "start")
  input_pos = _ffi.dev(input_pos, "input_pos")
  if start.dtype != torch.int32 or input_pos.dtype != torch.int32 or start.numel() != input_pos.numel():
    raise ValueError("start and input_pos must be int32 device tensors of one entry per slot")
  if cache_len % block_size != 0:
    raise ValueError("cache_len must be a multiple of block_size")
  batch = start.numel()
  b_next = torch.empty((batch, cache_len // block_size), dtype=torch.int32, device=start.device)
  i_next = torch.empty_like(b_next)
  _ffi.check(_ffi.lib.jpt_ragged_block_indices(
      _ffi.ptr(start.contiguous()), _ffi.ptr(input_pos.contiguous()), batch, int(cache_len), int(block_size),
      _ffi.ptr(b_next), _ffi.ptr(i_next), _ffi.stream()))
  return b_next, i_next
