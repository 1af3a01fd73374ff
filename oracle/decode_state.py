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
