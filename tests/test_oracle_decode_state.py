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
