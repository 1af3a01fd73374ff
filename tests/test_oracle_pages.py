"""Pins oracle.page_manager and the paged cache writer to the exact-integer
scenarios held by the reference's tests (tests/golden/reference_kats.json) and
to brute-force models."""

import queue

import numpy as np
import pytest
import torch

from oracle import Env
from oracle.kv_cache import KVCachePrefill, PageKVCacheGenerate
from oracle.page_manager import PageAttentionManager


def make_pam(cfg, **kw):
  return PageAttentionManager(
      cfg["batch_size"], cfg["total_num_pages"], cfg["page_size"],
      cfg["max_pages_per_sequence"], **kw)


def test_kat_reserve_pages_decode(kats):
  k = kats["pam_reserve_pages_decode"]
  pam = make_pam(k["manager"])
  for slot, n in k["insert"]:
    pam.reserve_pages_insert(slot, n)
  assert pam.page_indices[1][:2].tolist() == k["row1_after_insert_first2"]
  pam.fill_new_pages(np.asarray(k["fill_new_pages_lens"]))
  assert pam.page_indices[1].tolist() == k["row1_after_fill"]
  assert pam.page_indices[0].tolist() == k["row0_after_fill"]


def test_kat_get_page_token_indices(kats):
  k = kats["pam_get_page_token_indices"]
  pam = make_pam(k["manager"])
  for slot, n in k["insert"]:
    pam.reserve_pages_insert(slot, n)
  lens = np.asarray(k["lens"])
  pam.fill_new_pages(lens)
  pti = pam.get_page_token_indices(lens)
  assert pti[0].tolist() == k["expected_pages"]
  assert pti[1].tolist() == k["expected_tokens"]
  assert pti[2].tolist() == k["expected_slots"]
  assert pam.lengths.tolist() == k["expected_lengths_after"]


def _insert(pam, pages_k, pages_v, seq_len, dim, slot):
  kv = torch.arange(seq_len * dim).reshape(1, 1, seq_len, dim).to(torch.bfloat16)
  pre = KVCachePrefill()
  pre.update(kv, kv, 0)
  num_pages, idx = pam.reserve_pages_insert(slot, seq_len)
  pam.insert_prefill_cache([pre.state()], [(pages_k, pages_v)], idx)
  return num_pages


@pytest.mark.parametrize("name", ["prefill_insert", "prefill_insert_multiple_pages"])
def test_kat_prefill_insert(kats, name):
  k = kats[name]
  pam = make_pam(k["manager"])
  env = Env(paged_attention_total_num_pages=20, paged_attention_page_size=4)
  cache = PageKVCacheGenerate.empty(tuple(k["pages_shape"]), None, env)
  pk, pv = cache.state()
  _insert(pam, pk, pv, k["seq_len"], 2, k["slot"])
  for pages in (pk, pv):
    if name == "prefill_insert":
      assert pages[0, 0].tolist() == k["expected_page0"]
    else:
      assert pages[0, 0:2].tolist() == k["expected_pages_0_1"]
      lo, hi = k["untouched_pages"]
      assert torch.count_nonzero(pages[0, lo:hi]) == 0


def test_kat_page_attention_update(kats):
  k = kats["page_attention_update"]
  pam = make_pam(k["manager"])
  env = Env(paged_attention_total_num_pages=20, paged_attention_page_size=4)
  cache = PageKVCacheGenerate.empty(tuple(k["pages_shape"]), None, env)
  pk, pv = cache.state()
  for seq_len, slot in k["prefill_inserts_seq_len_slot"]:
    _insert(pam, pk, pv, seq_len, k["prefill_dim"], slot)
  lens = np.asarray(k["lens"])
  pam.fill_new_pages(lens)
  pti = pam.get_page_token_indices(lens)
  obj = PageKVCacheGenerate(pk, pv, pam, torch.from_numpy(pti), None, env=env)
  new = torch.arange(-1, -11, -1).reshape(5, 1, 1, 2).to(torch.bfloat16)
  rk, rv = obj.update(new, new)
  for pages in (rk, rv):
    assert pages[0, 0].tolist() == k["expected_page0"]
    assert pages[0, 7].tolist() == k["expected_page7"]
    assert pages[0, 6].tolist() == k["expected_page6"]


def test_paged_update_equals_direct_row_write():
  """The literal gather/set/scatter is the same as writing one row per active
  slot: pages[h, page_j, tok_j % ps, :] = new[slot_j, h, 0, :]."""
  g = torch.Generator().manual_seed(7)
  b, h, p, ps, d = 6, 3, 40, 8, 4
  pam = PageAttentionManager(b, p, ps, 5)
  lens = np.array([5, 0, 8, 17, 31, 1])
  for slot, n in enumerate(lens):
    if n:
      pam.reserve_pages_insert(slot, int(n))
  pages_k = torch.randn((h, p, ps, d), generator=g)
  pages_v = torch.randn((h, p, ps, d), generator=g)
  want_k, want_v = pages_k.clone(), pages_v.clone()
  pam.fill_new_pages(lens)
  pti = pam.get_page_token_indices(lens)
  nk = torch.randn((b, h, 1, d), generator=g)
  nv = torch.randn((b, h, 1, d), generator=g)
  for j in range(pti.shape[1]):
    page, tok, slot = (int(x) for x in pti[:, j])
    want_k[:, page, tok % ps, :] = nk[slot, :, 0, :]
    want_v[:, page, tok % ps, :] = nv[slot, :, 0, :]
  env = Env(paged_attention_total_num_pages=p, paged_attention_page_size=ps)
  env.bf16_enable = False
  obj = PageKVCacheGenerate(pages_k, pages_v, pam, torch.from_numpy(pti), None, env=env)
  obj.update(nk, nv)
  assert torch.equal(pages_k, want_k) and torch.equal(pages_v, want_v)


def test_allocator_against_bruteforce_model():
  """FIFO order, sentinel rows and conservation against a list model."""
  rng = np.random.default_rng(0)
  b, p, ps, mp = 8, 64, 4, 6
  order = rng.permutation(p)
  pam = PageAttentionManager(b, p, ps, mp, free_list_order=order)
  free = [int(x) for x in order]
  owned = {s: [] for s in range(b)}
  lens = np.zeros(b, dtype=np.int64)
  for _ in range(300):
    slot = int(rng.integers(b))
    if lens[slot] == 0 and rng.random() < 0.6:
      n = int(rng.integers(1, ps * 3))
      need = -(-n // ps)
      if need > len(free):
        with pytest.raises(queue.Empty):
          pam.reserve_pages_insert(slot, n)
        break
      k, row = pam.reserve_pages_insert(slot, n)
      owned[slot] = [free.pop(0) for _ in range(need)]
      assert k == need and row.tolist() == owned[slot]
      lens[slot] = n
    elif rng.random() < 0.3 and lens[slot]:
      pam.free_pages_resource(slot)
      free.extend(owned[slot])
      owned[slot], lens[slot] = [], 0
      assert pam.page_indices[slot].tolist() == [p - 1] * mp
    else:
      grow = [s for s in range(b) if lens[s] and lens[s] % ps == 0]
      if any(lens[s] // ps >= mp for s in grow) or len(grow) > len(free):
        continue
      pam.fill_new_pages(lens)
      for s in grow:
        owned[s].append(free.pop(0))
      pti = pam.get_page_token_indices(lens)
      act = [s for s in range(b) if lens[s]]
      assert pti[2].tolist() == act
      assert pti[0].tolist() == [owned[s][lens[s] // ps] for s in act]
      assert pti[1].tolist() == [j * ps + lens[s] % ps for j, s in enumerate(act)]
      lens = np.where(lens == 0, 0, lens + 1)
      assert pam.lengths.tolist() == lens.tolist()
    for s in range(b):
      assert pam.page_indices[s, :len(owned[s])].tolist() == owned[s]
    assert list(pam.unused_pages) == free
    everything = sorted(free + [x for s in owned.values() for x in s])
    assert everything == list(range(p))


def test_exhaustion_and_overflow():
  pam = PageAttentionManager(2, 3, 4, 2)
  pam.reserve_pages_insert(0, 8)
  with pytest.raises(queue.Empty):
    pam.reserve_pages_insert(1, 8)
  pam2 = PageAttentionManager(1, 8, 4, 2)
  pam2.reserve_pages_insert(0, 8)
  with pytest.raises(IndexError):
    pam2.fill_new_pages(np.array([8]))


def test_compress_cache_is_page_gather():
  g = torch.Generator().manual_seed(3)
  pam = PageAttentionManager(2, 16, 4, 4, free_list_order=[5, 9, 2, 11, 0, 1, 3, 4, 6, 7, 8, 10, 12, 13, 14, 15])
  pam.reserve_pages_insert(1, 10)
  pages = torch.randn((2, 16, 4, 3), generator=g)
  (k, v), = pam.get_compress_kv_cache([(pages, pages)], 1)
  want = torch.stack([torch.cat([pages[h, 5], pages[h, 9], pages[h, 2]])[:10] for h in range(2)])
  assert torch.equal(k, want) and torch.equal(v, want)
