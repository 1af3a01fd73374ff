"""The C++ page allocator (through the shipped Python class) against the oracle
and the reference's exact-integer scenarios.  Host code only: runs without a GPU."""

import queue

import numpy as np
import pytest

from jetstream_pt_amd.page_attention_manager import PageAttentionManager
from oracle.page_manager import PageAttentionManager as OraclePAM


def both(cfg, **kw):
  args = (cfg["batch_size"], cfg["total_num_pages"], cfg["page_size"], cfg["max_pages_per_sequence"])
  return PageAttentionManager(*args, **kw), OraclePAM(*args, **kw)


def test_kat_reserve_pages_decode(kats):
  k = kats["pam_reserve_pages_decode"]
  pam, _ = both(k["manager"])
  for slot, n in k["insert"]:
    num, row = pam.reserve_pages_insert(slot, n)
    assert num == 2 and row.tolist() == k["row1_after_insert_first2"]
  pam.fill_new_pages(np.asarray(k["fill_new_pages_lens"]))
  assert pam.page_indices[1].tolist() == k["row1_after_fill"]
  assert pam.page_indices[0].tolist() == k["row0_after_fill"]


def test_kat_get_page_token_indices(kats):
  k = kats["pam_get_page_token_indices"]
  pam, _ = both(k["manager"])
  for slot, n in k["insert"]:
    pam.reserve_pages_insert(slot, n)
  lens = np.asarray(k["lens"])
  pam.fill_new_pages(lens)
  pti = pam.get_page_token_indices(lens)
  assert pti.shape == (3, 3) and pti.dtype == np.int32
  assert pti[0].tolist() == k["expected_pages"]
  assert pti[1].tolist() == k["expected_tokens"]
  assert pti[2].tolist() == k["expected_slots"]
  assert pam.lengths.tolist() == k["expected_lengths_after"]


def test_row_view_aliases_the_table():
  pam = PageAttentionManager(2, 8, 4, 4)
  _, row = pam.reserve_pages_insert(1, 6)
  row[0] = 7  # a view, as in the reference
  assert pam.page_indices[1, 0] == 7


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_walk_matches_oracle(seed):
  rng = np.random.default_rng(seed)
  b, p, ps, mp = 16, 96, 8, 6
  order = rng.permutation(p).astype(np.int32)
  pam, ora = both(dict(batch_size=b, total_num_pages=p, page_size=ps, max_pages_per_sequence=mp),
                  free_list_order=order)
  lens = np.zeros(b, dtype=np.int32)
  for _ in range(400):
    slot = int(rng.integers(b))
    r = rng.random()
    if lens[slot] == 0 and r < 0.5:
      n = int(rng.integers(1, ps * (mp - 1)))
      if -(-n // ps) > len(ora.unused_pages):
        with pytest.raises(queue.Empty):
          pam.reserve_pages_insert(slot, n)
        continue
      k1, row1 = pam.reserve_pages_insert(slot, n)
      k2, row2 = ora.reserve_pages_insert(slot, n)
      assert k1 == k2 and row1.tolist() == row2.tolist()
      lens[slot] = n
    elif lens[slot] and r < 0.65:
      pam.free_pages_resource(slot)
      ora.free_pages_resource(slot)
      lens[slot] = 0
    else:
      grow = [s for s in range(b) if lens[s] and lens[s] % ps == 0]
      for s in grow:  # retire slots that filled their table row
        if lens[s] // ps >= mp:
          pam.free_pages_resource(s), ora.free_pages_resource(s)
          lens[s] = 0
      grow = [s for s in grow if lens[s]]
      if len(grow) > len(ora.unused_pages):
        continue
      pam.fill_new_pages(lens)
      ora.fill_new_pages(lens)
      a, o = pam.get_page_token_indices(lens), ora.get_page_token_indices(lens)
      assert a.tolist() == o.tolist()
      lens = np.where(lens == 0, 0, lens + 1).astype(np.int32)
    assert pam.page_indices.tolist() == ora.page_indices.tolist()
    assert pam.lengths.tolist() == list(ora.lengths)
    assert pam.unused_page_ids().tolist() == list(ora.unused_pages)


def test_conservation_after_free():
  pam = PageAttentionManager(4, 32, 4, 16)
  for slot, n in enumerate((5, 17, 32, 1)):
    pam.reserve_pages_insert(slot, n)
  pam.fill_new_pages(np.array([5, 17, 32, 1]))
  for slot in (2, 0, 3, 1):
    pam.free_pages_resource(slot)
  assert sorted(pam.unused_page_ids().tolist()) == list(range(32))
  assert np.all(pam.page_indices == 31) and np.all(pam.lengths == 0)
  # FIFO tail in free order, each slot's pages in row order: slot 2 held
  # pages 7..14 plus page 16, the boundary page fill_new_pages handed it
  assert pam.unused_page_ids().tolist()[-17:] == [7, 8, 9, 10, 11, 12, 13, 14, 16, 0, 1, 15, 2, 3, 4, 5, 6]


def test_errors_map_to_reference_exception_types():
  pam = PageAttentionManager(2, 3, 4, 2)
  pam.reserve_pages_insert(0, 8)
  with pytest.raises(queue.Empty):
    pam.reserve_pages_insert(1, 8)
  assert pam.lengths[1] == 0  # a refused insert leaves the slot untouched
  pam2 = PageAttentionManager(1, 8, 4, 2)
  pam2.reserve_pages_insert(0, 8)
  with pytest.raises(IndexError):
    pam2.fill_new_pages(np.array([8]))
  with pytest.raises(ValueError):
    pam2.reserve_pages_insert(5, 1)
  with pytest.raises(ValueError):
    PageAttentionManager(2, 4, 4, 2, free_list_order=[0, 1, 1, 2])
