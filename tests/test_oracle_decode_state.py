"""Pins oracle.decode_state (engine.py:774-812) by brute force and by the values
the reference's expressions fix."""
import numpy as np

from oracle import decode_state as ods


def test_update_mask_brute_force():
  rng = np.random.default_rng(1)
  mask = np.full((5, 9), -np.inf, dtype=np.float32)
  pos = rng.integers(0, 9, 5)
  got = ods.update_mask(mask, pos)
  for b in range(5):
    for s in range(9):
      assert got[b, s] == (0 if s == pos[b] else -np.inf)
  assert np.all(np.isinf(mask))  # the input is not touched
  ring = ods.update_mask(mask, pos, ring_buffer=True, current_position=4)
  assert np.all(ring[:, 4] == 0) and np.all(np.isinf(np.delete(ring, 4, axis=1)))


def test_advance_values():
  pos = np.array([0, 1, 7, 1023, 2047], dtype=np.int32)
  lens = np.array([0, 3, 7, 1, 2047], dtype=np.int32)
  p2, l2 = ods.advance(pos, lens, cache_len=2048)
  # position 0 marks an empty slot and stays; nothing wraps at cache_len
  assert p2.tolist() == [0, 2, 8, 1024, 2048] and l2.tolist() == [0, 4, 8, 2, 2048]
  p3, l3 = ods.advance(pos, lens, cache_len=2048, ring_buffer=True)
  assert p3.tolist() == [1, 2, 8, 1024, 2048] and l3.tolist() == [1, 4, 8, 2, 2048]


def _block_tables_by_positions(start, input_pos, cache_len, bk):
  """The tables stated through the live positions of each slot, position by
  position: a cell keeps its own block if the block holds a live position;
  a dead block in front of the live run (or inside the wrapped run's gap) jumps
  to the block of `start`; a block past the end of an unwrapped run, and every
  block of an empty slot, hands over to the next slot's block 0 - the last slot
  to itself, at the last block that can hold a live position."""
  batch, num_bk = len(start), cache_len // bk
  bn = np.zeros((batch, num_bk), dtype=np.int32)
  inn = np.zeros((batch, num_bk), dtype=np.int32)
  for b in range(batch):
    s = int(start[b])
    e = (s + int(input_pos[b])) % cache_len
    if s < e:
      live = set(range(s, e))
    elif s > e:
      live = set(range(s, cache_len)) | set(range(0, e))
    else:
      live = set()
    last = b == batch - 1
    if last:
      hand_b = b
      hand_i = max(p for p in range(s, e)) // bk if s < e else num_bk - 1
    else:
      hand_b, hand_i = b + 1, 0
    for i in range(num_bk):
      block = range(i * bk, (i + 1) * bk)
      if any(p in live for p in block):
        bn[b, i], inn[b, i] = b, i
      elif s == e or (s < e and i * bk >= e):
        bn[b, i], inn[b, i] = hand_b, hand_i
      else:
        bn[b, i], inn[b, i] = b, s // bk
  return bn, inn


def test_ragged_block_indices_brute_force():
  rng = np.random.default_rng(7)
  for cache_len, bk, batch in ((64, 16, 6), (128, 32, 5), (96, 8, 9), (32, 32, 3)):
    for _ in range(40):
      start = rng.integers(0, cache_len, batch)
      pos = rng.integers(0, cache_len, batch)
      # edge cases: block-aligned bounds, empty slots, runs that end at the cache end
      start[0] = (start[0] // bk) * bk
      pos[1] = 0
      pos[2] = (cache_len - start[2]) % cache_len
      got_b, got_i = ods.ragged_block_indices(start, pos, cache_len, bk)
      want_b, want_i = _block_tables_by_positions(start, pos, cache_len, bk)
      assert np.array_equal(got_b, want_b), (start, pos, got_b, want_b)
      assert np.array_equal(got_i, want_i), (start, pos, got_i, want_i)


def test_ragged_block_indices_left_aligned_case():
  # start = 0 everywhere (no ring buffer): blocks below the length stay, the
  # rest hand over to the next slot's block 0; the last slot to its own last block
  b_next, i_next = ods.ragged_block_indices([0, 0, 0], [5, 16, 40], cache_len=64, block_size=16)
  assert b_next.tolist() == [[0, 1, 1, 1], [1, 2, 2, 2], [2, 2, 2, 2]]
  assert i_next.tolist() == [[0, 0, 0, 0], [0, 0, 0, 0], [0, 1, 2, 2]]
