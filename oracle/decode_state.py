"""Per-step decode-state bookkeeping of generate_impl, restated (test infrastructure).

Follows jetstream_pt/engine.py:774-812.  Pinned by tests/test_oracle_kv_cache.py's
sibling tests/test_oracle_decode_state.py: brute-force loops and the values the
expressions fix (an inactive slot, position 0, stays at 0; `x + 1 % cache_len`
parses as x + (1 % cache_len), i.e. x + 1 for any cache longer than one).
"""

import numpy as np


def update_mask(mask, input_pos, ring_buffer=False, current_position=0):
  """engine.py:774-780: mask.at[:, current_position].set(0) with a ring
  buffer, else mask.at[arange(batch), input_pos].set(0).  Returns a copy."""
  out = np.array(mask, copy=True)
  if ring_buffer:
    out[:, current_position] = 0
  else:
    out[np.arange(out.shape[0]), np.asarray(input_pos)] = 0
  return out


def advance(input_pos, lens, cache_len, ring_buffer=False):
  """engine.py:800-812: the positions after a step."""
  input_pos, lens = np.asarray(input_pos), np.asarray(lens)
  if ring_buffer:
    return input_pos + 1, lens + 1
  return (np.where(input_pos == 0, 0, input_pos + 1 % cache_len),
          np.where(lens == 0, 0, lens + 1 % cache_len))


def ragged_block_indices(start, input_pos, cache_len, block_size):
  """engine.py:674-729: the (batch, cache_len // block_size) tables
  (b_next, i_next) that tell the reference's ring-aware ragged kernel, for grid
  cell (slot b, block i), which (slot, block) to work on.  The live ragged
  kernel of the reference ignores them (attention_kernel.py:561-579 calls the
  left-aligned one); restated for completeness, same where-expressions."""
  start = np.asarray(start).astype(np.int64)
  end = (start + np.asarray(input_pos).astype(np.int64)) % cache_len
  batch = start.shape[0]
  bk = block_size
  num_bk = cache_len // bk
  b = np.arange(batch).reshape(batch, 1)
  i = np.broadcast_to(np.arange(num_bk).reshape(1, num_bk), (batch, num_bk))
  start = start.reshape(batch, 1)
  end = end.reshape(batch, 1)
  last_slot = b == batch - 1
  last_good_block = np.where(start < end, (end - 1) // bk, (cache_len - 1) // bk)
  next_b = np.where(last_slot, b, b + 1)
  next_i = np.where(last_slot, last_good_block, 0)
  # start < end: stay while the block overlaps [start, end)
  past = i * bk >= end
  t_b = np.where(past, next_b, b)
  t_i = np.where(past, next_i, i)
  t_i = np.where((i + 1) * bk <= start, start // bk, t_i)
  # start > end: stay unless the block lies inside the gap [end, start)
  f_b = np.broadcast_to(b, (batch, num_bk))
  f_i = np.where((i * bk >= end) & ((i + 1) * bk <= start), start // bk, i)
  b_next = np.where(start < end, t_b, np.where(start == end, next_b, f_b))
  i_next = np.where(start < end, t_i, np.where(start == end, next_i, f_i))
  return b_next.astype(np.int32), i_next.astype(np.int32)
