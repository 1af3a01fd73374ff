"""Device-resident page allocator and decode-state bookkeeping against the oracle.

The allocator's tables are integers: every comparison is exact.  The oracle's
PageAttentionManager is pinned by the reference's own scenario
(tests/test_oracle_pages.py); here random request sequences drive both."""
import queue

import numpy as np
import pytest
import torch

from conftest import attention_bound
from oracle import decode_state as ods
from oracle.page_manager import PageAttentionManager as OPam

pytestmark = pytest.mark.gpu
DEV = "cuda"


def same_state(dp, op, what=""):
  assert np.array_equal(dp.page_indices.cpu().numpy(), op.page_indices), f"page table {what}"
  assert np.array_equal(dp.lengths.cpu().numpy(), np.asarray(op.lengths)), f"lengths {what}"
  assert dp.unused_page_ids().tolist() == list(op.unused_pages), f"free list {what}"


@pytest.mark.parametrize("batch,total,ps,mp,seed", [(5, 40, 4, 6, 0), (300, 4096, 16, 8, 1), (64, 512, 64, 4, 2)])
def test_random_request_sequences(batch, total, ps, mp, seed):
  from jetstream_pt_amd.page_attention_manager import DevicePageAttentionManager
  rng = np.random.default_rng(seed)
  order = rng.permutation(total).astype(np.int32)
  dp = DevicePageAttentionManager(batch, total, ps, mp, device=DEV, free_list_order=order)
  op = OPam(batch, total, ps, mp, free_list_order=order)
  same_state(dp, op, "after init")
  lens = np.zeros(batch, dtype=np.int32)
  dlens = torch.zeros(batch, dtype=torch.int32, device=DEV)
  for it in range(40):
    kind = rng.integers(0, 4)
    if kind == 0:  # a few inserts, one launch
      slots = rng.choice(batch, size=min(batch, 3), replace=False)
      slots = [s for s in slots if lens[s] == 0]
      ns = [int(rng.integers(1, ps * mp - 2 * ps)) for _ in slots]
      free_now = len(op.unused_pages)
      need = sum((n + ps - 1) // ps for n in ns)
      if not slots or need > free_now:
        continue
      for s, n in zip(slots, ns):
        op.reserve_pages_insert(int(s), n)
        lens[s] = n
      if len(slots) == 1:
        n, row = dp.reserve_pages_insert(int(slots[0]), ns[0])
        assert n == (ns[0] + ps - 1) // ps and row.shape == (n,)
        assert np.array_equal(row.cpu().numpy(), op.page_indices[slots[0], :n])
      else:
        dp.reserve_pages_insert_many(np.array(slots), np.array(ns))
      dlens.copy_(torch.from_numpy(lens))
    elif kind == 1:  # free some
      busy = np.flatnonzero(lens > 0)
      if busy.size == 0:
        continue
      slots = rng.choice(busy, size=min(busy.size, 2), replace=False)
      for s in slots:
        op.free_pages_resource(int(s))
        lens[s] = 0
      if len(slots) == 1:
        dp.free_pages_resource(int(slots[0]))
      else:
        dp.free_pages_resource_many(torch.tensor(slots, dtype=torch.int32, device=DEV))
      dlens.copy_(torch.from_numpy(lens))
    else:  # decode steps: allocate on page boundaries, index rows, advance
      for _ in range(int(rng.integers(1, 2 * ps))):
        growing = lens > 0
        if np.any(lens[growing] // ps >= mp - 1) or growing.sum() > len(op.unused_pages):
          break
        op.fill_new_pages(lens)
        want = op.get_page_token_indices(lens)
        got = dp.decode_step(dlens)
        host = got.to_host()
        assert host.shape == want.shape and np.array_equal(host, want), f"token indices, iteration {it}"
        lens = np.where(lens == 0, 0, lens + 1).astype(np.int32)
        from jetstream_pt_amd import decode_state
        decode_state.advance(dlens)
        assert np.array_equal(dlens.cpu().numpy(), lens)
    same_state(dp, op, f"iteration {it}")
  assert dp.status() == 0
  dp.check()


def test_failures_are_recorded_not_raised_and_stay_in_bounds():
  from jetstream_pt_amd.page_attention_manager import DevicePageAttentionManager
  dp = DevicePageAttentionManager(4, 6, 4, 3, device=DEV)
  dp.reserve_pages_insert(0, 12)   # 3 pages
  dp.reserve_pages_insert(1, 8)    # 2 pages, one left
  before = dp.page_indices.clone()
  dp.reserve_pages_insert(2, 9)    # needs 3: refused as a whole
  assert torch.equal(dp.page_indices, before) and dp.unused_page_ids().tolist() == [5]
  with pytest.raises(queue.Empty):
    dp.check()
  dp2 = DevicePageAttentionManager(2, 8, 4, 2, device=DEV)
  dp2.reserve_pages_insert(0, 8)
  lens = torch.tensor([8, 0], dtype=torch.int32, device=DEV)
  idx = dp2.decode_step(lens)      # slot 0 would need a third page of at most two
  assert int(idx.n_active.item()) == 1 and dp2.unused_page_ids().tolist() == [2, 3, 4, 5, 6, 7]
  with pytest.raises(IndexError):
    dp2.check()
  dp3 = DevicePageAttentionManager(2, 8, 4, 2, device=DEV)
  dp3.reserve_pages_insert_many(torch.tensor([5], device=DEV), torch.tensor([3], device=DEV))
  with pytest.raises(ValueError):
    dp3.check()
  with pytest.raises(ValueError):  # checked on the host for the single-request form
    dp3.reserve_pages_insert(7, 3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ring", [False, True])
def test_decode_state_bookkeeping(ring, dtype):
  from jetstream_pt_amd import decode_state
  rng = np.random.default_rng(3)
  b, s = 37, 129
  mask = torch.full((b, s), float("-inf"), dtype=dtype)
  pos = rng.integers(0, s, b).astype(np.int32)
  pos[:3] = 0
  lens = rng.integers(0, 50, b).astype(np.int32)
  want_mask = ods.update_mask(mask.float().numpy(), pos, ring, 17)
  want_pos, want_lens = ods.advance(pos, lens, s, ring)
  gm, gp, gl = mask.to(DEV), torch.from_numpy(pos).to(DEV), torch.from_numpy(lens).to(DEV)
  decode_state.finish_step(gm, gp, gl, ring_buffer=ring, current_position=17)
  assert np.array_equal(gm.float().cpu().numpy(), want_mask)
  assert np.array_equal(gp.cpu().numpy(), want_pos) and np.array_equal(gl.cpu().numpy(), want_lens)
  # the two halves separately, on a strided mask view
  wide = torch.full((b, 2 * s), float("-inf"), dtype=dtype, device=DEV)
  view = wide[:, :s]
  gp2 = torch.from_numpy(pos).to(DEV)
  decode_state.update_mask(view, gp2, ring_buffer=ring, current_position=17)
  assert np.array_equal(view.float().cpu().numpy(), want_mask) and torch.all(torch.isinf(wide[:, s:]))
  assert np.array_equal(gp2.cpu().numpy(), pos)
  decode_state.advance(gp2, ring_buffer=ring)
  assert np.array_equal(gp2.cpu().numpy(), want_pos)


@pytest.mark.parametrize("batch,cache_len,bk", [(6, 64, 16), (9, 96, 8), (128, 8192, 512), (1, 32, 32)])
def test_ragged_block_index_tables(batch, cache_len, bk):
  """engine.py:674-729 on the device: integer tables, exact."""
  from jetstream_pt_amd import decode_state
  rng = np.random.default_rng(batch + bk)
  for _ in range(5):
    start = rng.integers(0, cache_len, batch).astype(np.int32)
    pos = rng.integers(0, cache_len, batch).astype(np.int32)
    start[0] = (start[0] // bk) * bk
    pos[batch // 2] = 0  # an empty slot
    pos[-1] = (cache_len - start[-1]) % cache_len  # the last slot's run ends at the cache end
    want_b, want_i = ods.ragged_block_indices(start, pos, cache_len, bk)
    got_b, got_i = decode_state.ragged_block_indices(
        torch.from_numpy(start).to(DEV), torch.from_numpy(pos).to(DEV), cache_len, bk)
    assert got_b.shape == (batch, cache_len // bk)
    assert np.array_equal(got_b.cpu().numpy(), want_b) and np.array_equal(got_i.cpu().numpy(), want_i)
  # left-aligned slots (no ring buffer): start = 0
  zero = torch.zeros(batch, dtype=torch.int32, device=DEV)
  want_b, want_i = ods.ragged_block_indices(np.zeros(batch, np.int32), pos, cache_len, bk)
  got_b, got_i = decode_state.ragged_block_indices(zero, torch.from_numpy(pos).to(DEV), cache_len, bk)
  assert np.array_equal(got_b.cpu().numpy(), want_b) and np.array_equal(got_i.cpu().numpy(), want_i)
  with pytest.raises(ValueError):
    decode_state.ragged_block_indices(zero, zero, cache_len, bk + 1)


def _paged_setup(int8, seed):
  """Two identical paged caches, one driven by the host allocator, one by the
  device allocator, with the same prompts inserted."""
  from jetstream_pt_amd import cache_manager as cm
  from jetstream_pt_amd import insert as gins
  from jetstream_pt_amd.environment import JetEngineEnvironment, JetEngineEnvironmentData
  from jetstream_pt_amd.page_attention_manager import DevicePageAttentionManager, PageAttentionManager
  g = torch.Generator().manual_seed(seed)
  rng = np.random.default_rng(seed)
  b, hq, hkv, p, ps, d, mp = 9, 16, 4, 160, 32, 128, 10
  env = JetEngineEnvironment(JetEngineEnvironmentData(batch_size=b, paged_attention_total_num_pages=p,
                                                      paged_attention_page_size=ps))
  order = rng.permutation(p).astype(np.int32)
  hp = PageAttentionManager(b, p, ps, mp, free_list_order=order)
  dp = DevicePageAttentionManager(b, p, ps, mp, device=DEV, free_list_order=order)
  lens = np.array([31, 0, 32, 100, 1, 63, 0, 200, 64], dtype=np.int32)
  caches = []
  for pam in (hp, dp):
    if int8:
      c = cm.Int8PageKVCacheGenerate.empty((hkv, p, ps, d), DEV, env)
      c.page_attention_manager = pam
    else:
      c = cm.PageKVCacheGenerate.empty((hkv, p, ps, d), DEV, env)
      c.page_attention_manager = pam
    caches.append(c)
  for slot, n in enumerate(lens):
    if not n:
      continue
    k = torch.randn((1, hkv, int(n), d), generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn((1, hkv, int(n), d), generator=g).to(torch.bfloat16).to(DEV)
    for pam, c in zip((hp, dp), caches):
      _, ids = pam.reserve_pages_insert(slot, int(n))
      if int8:
        gins.insert_prefix_pages_int8([(k, v)], [(c.cache_k, c.cache_v)], [(c.k_scaler, c.v_scaler)], ids)
      else:
        pam.insert_prefill_cache([(k, v)], [(c.cache_k, c.cache_v)], ids)
  return env, hp, dp, caches, lens, (b, hq, hkv, d), g


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("int8", [False, True])
def test_paged_decode_steps_device_allocator_equals_host_allocator(int8, fused):
  """Whole decode steps - page allocation, token indices, (quantised) paged
  append, paged attention, position advance - with nothing crossing to the
  host, eagerly and as replays of one captured HIP graph; pages, scale pages
  and tables must equal the host-allocator flow bit for bit.  fused: the
  device flow's attention launch appends (and quantises) the token itself - no
  append launch; its outputs sum in another order, so they are held to the
  attention tolerance instead of bit equality."""
  from jetstream_pt_amd import decode_state, layers
  env, hp, dp, (hc, dc), lens, (b, hq, hkv, d), g = _paged_setup(int8, 401 + int(int8))
  cls = layers.Int8KVAttentionKernel if int8 else layers.AttentionKernel
  kern_h = cls(env, 0, fuse_new_token=False)
  kern = cls(env, 0, fuse_new_token=fused)
  dlens = torch.from_numpy(lens).to(DEV)
  xq = torch.empty((b, hq, 1, d), dtype=torch.bfloat16, device=DEV)
  xk = torch.empty((b, hkv, 1, d), dtype=torch.bfloat16, device=DEV)
  xv = torch.empty_like(xk)
  out_d = torch.empty_like(xq)

  def device_step():
    dc.page_token_indices = dp.decode_step(dlens)
    assert kern._will_append_in_launch(xq, dc, dc.cache_k) == fused
    out_d.copy_(kern(xq, xk, xv, None, dc))
    decode_state.advance(dlens)

  def host_step():
    nonlocal lens
    hp.fill_new_pages(lens)
    hc.page_token_indices = torch.from_numpy(hp.get_page_token_indices(lens)).to(DEV)
    out = kern_h(xq, xk, xv, None, hc)
    lens = np.where(lens == 0, 0, lens + 1).astype(np.int32)
    return out

  def same_output(got, want, what):
    if not fused:
      assert torch.equal(got, want), what
      return
    live = torch.from_numpy(lens > 0).to(DEV)  # inactive slots: nothing is attended
    # `want` is the separate launches' bf16 output: half an ulp of its own on top
    err = (got.float() - want.float()).abs()[live]
    assert torch.all(err <= attention_bound(want.float(), rounded_want=True)[live]), f"{what}: max err {err.max():.4g}"

  def new_inputs():
    for t in (xq, xk, xv):
      t.copy_(torch.randn(t.shape, generator=g).to(torch.bfloat16))

  def compare(what):
    assert torch.equal(dc.cache_k, hc.cache_k) and torch.equal(dc.cache_v, hc.cache_v), f"pages, {what}"
    if int8:
      assert torch.equal(dc.k_scaler, hc.k_scaler) and torch.equal(dc.v_scaler, hc.v_scaler), f"scale pages, {what}"
    assert np.array_equal(dp.page_indices.cpu().numpy(), hp.page_indices), f"page table, {what}"
    assert np.array_equal(dp.lengths.cpu().numpy(), hp.lengths), f"lengths, {what}"
    assert np.array_equal(dlens.cpu().numpy(), lens), f"lens, {what}"

  for step in range(3):  # eager; also warms every launch up before capture
    new_inputs()
    want = host_step()
    device_step()
    same_output(out_d, want, f"eager step {step}")
    compare(f"eager step {step}")
  graph = torch.cuda.CUDAGraph()
  snapshot = [t.clone() for t in (dp._mem, dlens, dc.cache_k, dc.cache_v)] + (
      [dc.k_scaler.clone(), dc.v_scaler.clone()] if int8 else [])
  with torch.cuda.graph(graph):
    device_step()
  # capture ran nothing: restore is not needed, but make sure of it
  for t, s in zip([dp._mem, dlens, dc.cache_k, dc.cache_v] + ([dc.k_scaler, dc.v_scaler] if int8 else []), snapshot):
    assert torch.equal(t, s)
  for step in range(40):  # crosses a page boundary for every live slot (page size 32)
    new_inputs()
    want = host_step()
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    same_output(out_d, want, f"replay {step}")
    compare(f"replay {step}")
  dp.check()


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("int8", [False, True])
def test_a_decode_step_without_a_free_page_drops_the_token_and_touches_no_other_page(int8, fused):
  """The pool runs out in a decode step (the reference raises queue.Empty before
  anything is written, page_attention_manager.py:55-64).  On the device the
  slots that were served get their pages as usual; a slot that was not gets page
  id -1 in its index column and table cell, its length stays, and no page -
  in particular none that belongs to another slot, and not the sentinel page -
  receives its token, with a separate append launch or with the attention launch
  appending.  check() raises queue.Empty once and clears the record."""
  from jetstream_pt_amd import cache_manager as cm
  from jetstream_pt_amd import layers
  from jetstream_pt_amd.environment import JetEngineEnvironment, JetEngineEnvironmentData
  from jetstream_pt_amd.page_attention_manager import DevicePageAttentionManager
  g = torch.Generator().manual_seed(77 + int(int8) + 2 * int(fused))
  b, hq, hkv, p, ps, d, mp = 4, 8, 2, 9, 32, 128, 4
  env = JetEngineEnvironment(JetEngineEnvironmentData(batch_size=b, paged_attention_total_num_pages=p,
                                                      paged_attention_page_size=ps))
  dp = DevicePageAttentionManager(b, p, ps, mp, device=DEV)
  cache = (cm.Int8PageKVCacheGenerate if int8 else cm.PageKVCacheGenerate).empty((hkv, p, ps, d), DEV, env)
  cache.page_attention_manager = dp
  # 2 + 2 + 2 + 1 pages taken, two left (the last of them is the sentinel id 8);
  # slots 0, 1 and 2 all sit on a page boundary: three requests for two pages
  lens = np.array([64, 64, 64, 5], dtype=np.int32)
  dp.reserve_pages_insert_many(np.arange(b, dtype=np.int32), lens)
  for t in (cache.cache_k, cache.cache_v):
    if int8:
      t.random_(-127, 128)
    else:
      t.normal_()
  if int8:
    cache.k_scaler.uniform_(0.01, 0.05)
    cache.v_scaler.uniform_(0.01, 0.05)
  dlens = torch.from_numpy(lens).to(DEV)
  table_before = dp.page_indices.clone()
  saved = [t.clone() for t in ((cache.cache_k, cache.cache_v) + ((cache.k_scaler, cache.v_scaler) if int8 else ()))]
  xq = torch.randn((b, hq, 1, d), generator=g).to(torch.bfloat16).to(DEV)
  xk = torch.randn((b, hkv, 1, d), generator=g).to(torch.bfloat16).to(DEV)
  xv = torch.randn((b, hkv, 1, d), generator=g).to(torch.bfloat16).to(DEV)
  kern = (layers.Int8KVAttentionKernel if int8 else layers.AttentionKernel)(env, 0, fuse_new_token=fused)
  cache.page_token_indices = dp.decode_step(dlens)
  assert kern._will_append_in_launch(xq, cache, cache.cache_k) == fused
  kern(xq, xk, xv, None, cache)
  torch.cuda.synchronize()
  idx = cache.page_token_indices.to_host()
  assert idx[2].tolist() == [0, 1, 2, 3]
  assert idx[0].tolist() == [7, 8, -1, int(table_before[3, 0])]          # slots 0, 1 served in order, slot 2 not
  assert dp.lengths.cpu().tolist() == [65, 65, 64, 6]
  table = dp.page_indices.cpu()
  assert table[0, 2] == 7 and table[1, 2] == 8 and table[2, 2] == -1
  assert dp.unused_page_ids().tolist() == []
  # pages: exactly the rows (page 7, 0), (page 8, 0) and (slot 3's page, 5) changed
  now = (cache.cache_k, cache.cache_v) + ((cache.k_scaler, cache.v_scaler) if int8 else ())
  written = [(7, 0), (8, 0), (int(table_before[3, 0]), 5)]
  for before, after in zip(saved, now):
    changed = (before != after)
    while changed.dim() > 3:
      changed = changed.any(dim=-1)
    changed = changed.any(dim=0)  # (pages, rows in a page)
    assert sorted(map(tuple, changed.nonzero().tolist())) == sorted(written)
  with pytest.raises(queue.Empty):
    dp.check()
  dp.check()  # the record was cleared
